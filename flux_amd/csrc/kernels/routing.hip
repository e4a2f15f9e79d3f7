// Routing: stable counting sort of (token, k) pairs by expert id -> splits, offsets, scatter_index,
// gather_index, topk_index.
//
// The flat pair array is cut into chunks of kChunk = 512 pairs, one wave per chunk (8 wave-steps of 64).
// Inputs of up to 4096 pairs and 512 experts run the same three steps inside one workgroup
// (route_sort_single_kernel); larger ones take these steps:
//   1. route_hist_kernel    per-chunk expert histogram in LDS (ds_add_u32), written to hist[chunk][e]
//   2. route_scan_kernel    one wave per expert: exclusive scan of hist[:, e] over chunks (wave scan),
//                           in place; the total is splits[e]
//   3. route_scatter_kernel per chunk: running[e] = offsets[e] + base[chunk][e] in LDS; for each
//                           wave-step the lanes holding the same expert are found with ballots over the
//                           bits of the id, ranked with mbcnt, and the first of them advances running[e].
// Up to 256 chunks (131072 pairs) step 2 is folded into step 3 (each scatter workgroup sums the histogram
// columns it needs from L2): two launches instead of three, and launch gaps are most of the time at these sizes.
// Every pair is read twice (8 B) and each output written once: the array traffic is the whole cost.
#include "common.hpp"

namespace fluxmi {
namespace {

constexpr int kChunk = 512;           // pairs per wave
constexpr int kWavesPerBlock = 4;
constexpr int kThreads = kWavesPerBlock * 64;
constexpr int kMaxExperts = 1024;
// Up to this many chunks (131072 pairs) the scatter kernel scans the per-chunk histograms itself (two launches);
// beyond, a scan kernel of its own prepares them (three): the fused scan reads the table once per workgroup.
constexpr int kFusedScanMaxChunks = 256;

__global__ __launch_bounds__(kThreads) void route_hist_kernel(const int32_t *__restrict__ choosed,
                                                              int32_t npairs, int32_t nexperts,
                                                              int32_t nchunks,
                                                              int32_t *__restrict__ hist) {
  extern __shared__ int32_t s_hist[];  // [kWavesPerBlock][nexperts]
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  for (int i = threadIdx.x; i < kWavesPerBlock * nexperts; i += kThreads) s_hist[i] = 0;
  __syncthreads();
  const int chunk = blockIdx.x * kWavesPerBlock + wave;
  int32_t *my = s_hist + wave * nexperts;
  if (chunk < nchunks) {
    const int base = chunk * kChunk;
#pragma unroll
    for (int s = 0; s < kChunk / 64; ++s) {
      const int i = base + s * 64 + lane;
      if (i < npairs) {
        const int32_t e = choosed[i];
        if (e >= 0 && e < nexperts) atomicAdd(&my[e], 1);
      }
    }
  }
  __syncthreads();
  if (chunk < nchunks) {
    for (int e = lane; e < nexperts; e += 64) hist[static_cast<size_t>(chunk) * nexperts + e] = my[e];
  }
}

// grid = ceil(E / 4) blocks of 4 waves; wave -> expert.
__global__ __launch_bounds__(kThreads) void route_scan_kernel(int32_t *__restrict__ hist,
                                                              int32_t nexperts, int32_t nchunks,
                                                              int32_t *__restrict__ splits_ws,
                                                              int32_t *__restrict__ splits_out) {
  const int e = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (e >= nexperts) return;
  int running = 0;
  for (int c0 = 0; c0 < nchunks; c0 += 64) {
    const int c = c0 + lane;
    const int v = c < nchunks ? hist[static_cast<size_t>(c) * nexperts + e] : 0;
    const int incl = wave_inclusive_scan(v);
    if (c < nchunks) hist[static_cast<size_t>(c) * nexperts + e] = running + incl - v;
    running += __shfl(incl, 63, 64);
  }
  if (lane == 0) {
    splits_ws[e] = running;
    if (splits_out) splits_out[e] = running;
  }
}

// Stable scatter of the pairs [first, first + 64*steps) by one wave.  running[e] holds the next free
// sorted row of expert e for this range (LDS, private to the wave).  Per wave-step the lanes holding the
// same expert are found with one ballot per id bit, ranked with mbcnt, and the first of them advances
// running[e].
template <bool STAGED>
__device__ __forceinline__ void scatter_range(const int32_t *__restrict__ choosed, const uint16_t *staged,
                                              int first, int steps,
                                              int32_t npairs, int32_t topk, int32_t nexperts, int32_t idbits,
                                              int32_t *running, int32_t *__restrict__ scatter_index,
                                              int32_t *__restrict__ gather_index,
                                              int32_t *__restrict__ topk_index) {
  const int lane = threadIdx.x & 63;
  // Expert ids are fetched several wave-steps at a time.  From global memory all 8 steps of a chunk are
  // fetched before the first store: vmcnt counts loads and stores in one queue, so a later load would
  // also wait for every store issued before it.
  constexpr int kAhead = STAGED ? 4 : 8;
  int32_t ids[kAhead];
  for (int s = 0; s < steps; ++s) {
    if ((s & (kAhead - 1)) == 0) {
#pragma unroll
      for (int a = 0; a < kAhead; ++a) {
        const int ia = first + (s + a) * 64 + lane;
        if constexpr (STAGED) ids[a] = (s + a < steps && ia < npairs) ? static_cast<int32_t>(staged[ia]) : -1;
        else ids[a] = (s + a < steps && ia < npairs) ? choosed[ia] : -1;
      }
    }
    const int i = first + s * 64 + lane;
    int32_t e = ids[0];
#pragma unroll
    for (int a = 1; a < kAhead; ++a)
      if ((s & (kAhead - 1)) == a) e = ids[a];
    if (e < 0 || e >= nexperts) e = -1;
    // Lanes that hold the same expert id as this lane.
    uint64_t same = __ballot(e >= 0);
    for (int b = 0; b < idbits; ++b) {
      const uint64_t bit = __ballot((e >> b) & 1);
      same &= ((e >> b) & 1) ? bit : ~bit;
    }
    if (e >= 0) {
      const int rank = popc_below_lane(same);
      const int start = running[e];
      __builtin_amdgcn_wave_barrier();
      if (rank == 0) running[e] = start + __popcll(same);
      const int row = start + rank;
      scatter_index[i] = row;
      if (gather_index) gather_index[row] = i / topk;
      if (topk_index) topk_index[row] = i % topk;
    } else {
      __builtin_amdgcn_wave_barrier();
      if (i < npairs) scatter_index[i] = -1;
    }
    __builtin_amdgcn_wave_barrier();
  }
}

// FUSED_SCAN: `base` holds the raw per-chunk histograms and every workgroup sums, per expert, the chunks ahead
// of its own four (their starting offsets) and all chunks (the expert's total), so that the scan kernel and its
// launch gap disappear; hist is chunks x experts int32 and sits in L2.  Used while that table is small.
template <bool FUSED_SCAN>
__global__ __launch_bounds__(kThreads) void route_scatter_kernel(
    const int32_t *__restrict__ choosed, int32_t npairs, int32_t topk, int32_t nexperts,
    int32_t nchunks, int32_t idbits, const int32_t *__restrict__ base,
    const int32_t *__restrict__ splits_ws, int32_t *__restrict__ splits_out, int32_t *__restrict__ offsets_out,
    int32_t *__restrict__ scatter_index, int32_t *__restrict__ gather_index,
    int32_t *__restrict__ topk_index) {
  extern __shared__ int32_t s_mem[];  // [nexperts] offsets, [kWavesPerBlock][nexperts] running, FUSED: [2][nexperts] totals, sums ahead
  int32_t *s_off = s_mem;
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  int32_t *running = s_mem + nexperts + wave * nexperts;
  int32_t *s_tot = s_mem + (1 + kWavesPerBlock) * nexperts;
  const int chunk0 = blockIdx.x * kWavesPerBlock;

  if constexpr (FUSED_SCAN) {
    // Column sums of the chunks x experts table, per expert: over the chunks ahead of this workgroup's four (s_before)
    // and over all chunks (s_tot).  All lanes sweep the table in its memory order (coalesced, independent loads, four
    // in flight per lane) and add into LDS; the table is small (C4: 192 x 64) and sits in L2.
    int32_t *s_before = s_tot + nexperts;
    for (int e = threadIdx.x; e < nexperts; e += kThreads) {
      s_tot[e] = 0;
      s_before[e] = 0;
    }
    __syncthreads();
    const int total = nchunks * nexperts;
    const int before_end = (chunk0 < nchunks ? chunk0 : nchunks) * nexperts;
    for (int f0 = threadIdx.x; f0 < total; f0 += 4 * kThreads) {
      int32_t v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int f = f0 + u * kThreads;
        v[u] = f < total ? base[f] : 0;
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int f = f0 + u * kThreads;
        if (v[u] != 0) {
          const int e = f % nexperts;
          atomicAdd(&s_tot[e], v[u]);
          if (f < before_end) atomicAdd(&s_before[e], v[u]);
        }
      }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < nexperts; e += kThreads) {
      int sum = s_before[e];
#pragma unroll
      for (int w = 0; w < kWavesPerBlock; ++w) {
        s_mem[nexperts + w * nexperts + e] = sum;  // rows of expert e in the chunks ahead of chunk0 + w
        if (chunk0 + w < nchunks) sum += base[static_cast<size_t>(chunk0 + w) * nexperts + e];
      }
      if (blockIdx.x == 0 && splits_out) splits_out[e] = s_tot[e];
    }
    __syncthreads();
  }

  // Exclusive prefix sum of splits -> offsets (every block recomputes it; E <= 1024).
  if (wave == 0) {
    int carry = 0;
    for (int e0 = 0; e0 < nexperts; e0 += 64) {
      const int e = e0 + lane;
      const int v = e < nexperts ? (FUSED_SCAN ? s_tot[e] : splits_ws[e]) : 0;
      const int incl = wave_inclusive_scan(v);
      if (e < nexperts) s_off[e] = carry + incl - v;
      carry += __shfl(incl, 63, 64);
    }
    if (blockIdx.x == 0 && offsets_out) {
      for (int e = lane; e < nexperts; e += 64) offsets_out[e] = s_off[e];
      if (lane == 0) offsets_out[nexperts] = carry;
    }
  }
  __syncthreads();

  const int chunk = chunk0 + wave;
  if (chunk >= nchunks) return;
  for (int e = lane; e < nexperts; e += 64)
    running[e] = s_off[e] + (FUSED_SCAN ? running[e] : base[static_cast<size_t>(chunk) * nexperts + e]);
  __builtin_amdgcn_wave_barrier();

  scatter_range<false>(choosed, nullptr, chunk * kChunk, kChunk / 64, npairs, topk, nexperts, idbits, running,
                       scatter_index, gather_index, topk_index);
}

// Whole sort in one launch for small inputs: one workgroup of 16 waves, wave w owns the contiguous pair
// range [w*span, (w+1)*span).  The expert ids are first copied into LDS as 16-bit values by all 1024
// lanes at once (one coalesced sweep; out-of-range ids become 0xffff), so that the two ordered passes
// never wait on global memory.  LDS: hist[16][E] (becomes the per-wave running offsets), tot[E], off[E],
// ids[npairs].
constexpr int kSingleWaves = 16;
constexpr int kSingleMaxPairs = 4096;  // beyond this the scattered index stores of one CU become the limit
constexpr int kSingleMaxExperts = 512;

__global__ __launch_bounds__(kSingleWaves * 64) void route_sort_single_kernel(
    const int32_t *__restrict__ choosed, int32_t npairs, int32_t topk, int32_t nexperts, int32_t idbits,
    int32_t *__restrict__ splits_out, int32_t *__restrict__ offsets_out, int32_t *__restrict__ scatter_index,
    int32_t *__restrict__ gather_index, int32_t *__restrict__ topk_index) {
  extern __shared__ int32_t s_mem[];
  int32_t *s_hist = s_mem;                              // [kSingleWaves][nexperts]
  int32_t *s_tot = s_mem + kSingleWaves * nexperts;     // [nexperts]
  int32_t *s_off = s_tot + nexperts;                    // [nexperts]
  uint16_t *s_ids = reinterpret_cast<uint16_t *>(s_off + nexperts);  // [npairs]
  for (int i = threadIdx.x; i < npairs; i += blockDim.x) {
    const int32_t e = choosed[i];
    s_ids[i] = (e >= 0 && e < nexperts) ? static_cast<uint16_t>(e) : static_cast<uint16_t>(0xffff);
  }
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int steps = ((npairs + kSingleWaves - 1) / kSingleWaves + 63) / 64;  // wave-steps per wave
  const int first = wave * steps * 64;
  for (int i = threadIdx.x; i < kSingleWaves * nexperts; i += blockDim.x) s_hist[i] = 0;
  __syncthreads();
  int32_t *my = s_hist + wave * nexperts;
  for (int s = 0; s < steps; ++s) {
    const int i = first + s * 64 + lane;
    if (i < npairs) {
      const int32_t e = s_ids[i];
      if (e < nexperts) atomicAdd(&my[e], 1);
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < nexperts; e += blockDim.x) {
    int run = 0;
#pragma unroll
    for (int w = 0; w < kSingleWaves; ++w) {
      const int t = s_hist[w * nexperts + e];
      s_hist[w * nexperts + e] = run;
      run += t;
    }
    s_tot[e] = run;
    if (splits_out) splits_out[e] = run;
  }
  __syncthreads();
  if (wave == 0) {
    int carry = 0;
    for (int e0 = 0; e0 < nexperts; e0 += 64) {
      const int e = e0 + lane;
      const int v = e < nexperts ? s_tot[e] : 0;
      const int incl = wave_inclusive_scan(v);
      if (e < nexperts) {
        s_off[e] = carry + incl - v;
        if (offsets_out) offsets_out[e] = carry + incl - v;
      }
      carry += __shfl(incl, 63, 64);
    }
    if (lane == 0 && offsets_out) offsets_out[nexperts] = carry;
  }
  __syncthreads();
  for (int e = lane; e < nexperts; e += 64) my[e] += s_off[e];
  __builtin_amdgcn_wave_barrier();
  scatter_range<true>(choosed, s_ids, first, steps, npairs, topk, nexperts, idbits, my, scatter_index,
                      gather_index, topk_index);
}

__global__ __launch_bounds__(256) void gather_index_kernel(const int32_t *__restrict__ scatter_index,
                                                           int32_t npairs, int32_t nrows,
                                                           int32_t topk,
                                                           int32_t *__restrict__ gather_index,
                                                           int32_t *__restrict__ topk_index) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= npairs) return;
  const int32_t row = scatter_index[i];
  if (row < 0 || row >= nrows) return;
  gather_index[row] = i / topk;
  if (topk_index) topk_index[row] = i % topk;
}

inline int32_t num_chunks(int64_t npairs) { return static_cast<int32_t>((npairs + kChunk - 1) / kChunk); }

}  // namespace
}  // namespace fluxmi

extern "C" size_t fluxmi_moe_route_sort_workspace_bytes(int32_t ntokens, int32_t topk,
                                                        int32_t nexperts) {
  using namespace fluxmi;
  if (ntokens < 0 || topk < 1 || nexperts < 1) return 0;
  const int64_t npairs = static_cast<int64_t>(ntokens) * topk;
  const int64_t nchunks = num_chunks(npairs) > 0 ? num_chunks(npairs) : 1;
  return static_cast<size_t>((nchunks + 1) * nexperts) * sizeof(int32_t);
}

namespace fluxmi {
namespace {

// The sort itself on a workspace of at least fluxmi_moe_route_sort_workspace_bytes() bytes.  Nothing in the
// workspace has to be zero on entry: the histogram kernel writes every hist[chunk][expert] entry (and the scan
// kernel every splits entry) before anything reads them.
int route_sort_on_workspace(const int32_t *choosed, int32_t ntokens, int32_t topk,
                            int32_t nexperts, int32_t *splits, int32_t *offsets, int32_t *scatter_index,
                            int32_t *gather_index, int32_t *topk_index, void *workspace, void *stream) {
  const int32_t npairs = ntokens * topk;
  const int32_t nchunks = num_chunks(npairs);
  hipStream_t s = static_cast<hipStream_t>(stream);
  int32_t *splits_ws = static_cast<int32_t *>(workspace);
  int32_t *hist = splits_ws + nexperts;
  int idbits = 0;
  while ((1 << idbits) < nexperts) ++idbits;

  if (npairs <= kSingleMaxPairs && nexperts <= kSingleMaxExperts) {
    static std::atomic<uint64_t> lds_done{0};
    const int rc = ensure_dynamic_lds(reinterpret_cast<const void *>(route_sort_single_kernel), 128 * 1024, lds_done);
    if (rc != FLUXMI_OK) return rc;
    hipLaunchKernelGGL(route_sort_single_kernel, dim3(1), dim3(kSingleWaves * 64),
                       (kSingleWaves + 2) * nexperts * sizeof(int32_t) + ((npairs + 1) & ~1) * sizeof(uint16_t), s, choosed, npairs, topk, nexperts, idbits,
                       splits, offsets, scatter_index, gather_index, topk_index);
    FLUXMI_HIP_CHECK(hipGetLastError());
    return FLUXMI_OK;
  }
  const unsigned nblocks = static_cast<unsigned>((nchunks + kWavesPerBlock - 1) / kWavesPerBlock);
  if (nchunks > 0) {
    hipLaunchKernelGGL(route_hist_kernel, dim3(nblocks), dim3(kThreads),
                       kWavesPerBlock * nexperts * sizeof(int32_t), s, choosed, npairs, nexperts,
                       nchunks, hist);
  }
  if (nchunks <= kFusedScanMaxChunks) {
    // Two launches: every scatter workgroup scans the histogram table itself.  With no pairs one block still
    // runs to publish splits and offsets (all zero).
    hipLaunchKernelGGL(route_scatter_kernel<true>, dim3(nblocks > 0 ? nblocks : 1), dim3(kThreads),
                       (3 + kWavesPerBlock) * nexperts * sizeof(int32_t), s, choosed, npairs, topk, nexperts, nchunks,
                       idbits, hist, splits_ws, splits, offsets, scatter_index, gather_index, topk_index);
  } else {
    hipLaunchKernelGGL(route_scan_kernel, dim3((nexperts + kWavesPerBlock - 1) / kWavesPerBlock),
                       dim3(kThreads), 0, s, hist, nexperts, nchunks, splits_ws, splits);
    hipLaunchKernelGGL(route_scatter_kernel<false>, dim3(nblocks > 0 ? nblocks : 1), dim3(kThreads),
                       (1 + kWavesPerBlock) * nexperts * sizeof(int32_t), s, choosed, npairs, topk, nexperts, nchunks,
                       idbits, hist, splits_ws, splits, offsets, scatter_index, gather_index, topk_index);
  }
  FLUXMI_HIP_CHECK(hipGetLastError());
  return FLUXMI_OK;
}

// Argument checks shared by the entry points.
int route_sort_check(const char *who, const int32_t *choosed, int32_t ntokens, int32_t topk, int32_t nexperts,
                     const int32_t *scatter_index) {
  FLUXMI_REQUIRE(ntokens >= 0 && topk >= 1, FLUXMI_ERR_INVALID_ARG, "%s: bad sizes (ntokens=%d, topk=%d)", who,
                 ntokens, topk);
  FLUXMI_REQUIRE(nexperts >= 1 && nexperts <= kMaxExperts, FLUXMI_ERR_UNSUPPORTED,
                 "%s: nexperts=%d outside [1,%d]", who, nexperts, kMaxExperts);
  const int64_t npairs64 = static_cast<int64_t>(ntokens) * topk;
  FLUXMI_REQUIRE(npairs64 <= (int64_t{1} << 30), FLUXMI_ERR_UNSUPPORTED, "%s: ntokens*topk=%lld exceeds 2^30", who,
                 static_cast<long long>(npairs64));
  FLUXMI_REQUIRE((scatter_index != nullptr && choosed != nullptr) || npairs64 == 0, FLUXMI_ERR_INVALID_ARG,
                 "%s: null choosed / scatter_index", who);
  return FLUXMI_OK;
}

}  // namespace
}  // namespace fluxmi

extern "C" int fluxmi_moe_route_sort(const int32_t *choosed, int32_t ntokens, int32_t topk,
                                     int32_t nexperts, int32_t *splits, int32_t *offsets,
                                     int32_t *scatter_index, int32_t *gather_index,
                                     int32_t *topk_index, void *workspace, size_t workspace_bytes,
                                     void *stream) {
  using namespace fluxmi;
  const int rc = route_sort_check("moe_route_sort", choosed, ntokens, topk, nexperts, scatter_index);
  if (rc != FLUXMI_OK) return rc;
  const size_t need = fluxmi_moe_route_sort_workspace_bytes(ntokens, topk, nexperts);
  FLUXMI_REQUIRE(workspace != nullptr && workspace_bytes >= need, FLUXMI_ERR_WORKSPACE,
                 "moe_route_sort: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
  return route_sort_on_workspace(choosed, ntokens, topk, nexperts, splits, offsets, scatter_index,
                                 gather_index, topk_index, workspace, stream);
}

// ---- entry point that allocates nothing --------------------------------------------------------------------
// The sort's scratch (per-chunk histograms) in a file-scope device array instead of a caller's workspace, for
// callers that cannot allocate.  Every GPU holds its own copy of the array at its own address; the address is
// looked up once per device and kept.  In host code the array's name is only a handle for that lookup.
namespace fluxmi {
namespace {

constexpr size_t kStaticScratchBytes = size_t{4} << 20;  // 4 MiB per GPU, held until the process ends
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

std::atomic<void *> g_scratch_ptr[64];  // device id -> device address of `scratch` on that GPU
// device id -> event recorded behind the last eager call on that GPU.  The next eager call's stream waits for it, so
// that calls issued one after the other from different streams run one after the other on the shared array instead
// of racing.  (Host threads that call at the same moment, and replays of a captured graph against eager calls, are
// still the caller's to order.)
std::atomic<hipEvent_t> g_scratch_event[64];

int static_scratch(void **out, int *dev_out) {
  int dev = 0;
  FLUXMI_HIP_CHECK(hipGetDevice(&dev));
  FLUXMI_REQUIRE(dev >= 0 && dev < 64, FLUXMI_ERR_UNSUPPORTED, "moe_route_sort_static: device id %d outside [0,64)", dev);
  void *ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (ptr == nullptr) {
    FLUXMI_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    FLUXMI_REQUIRE(ptr != nullptr, FLUXMI_ERR_HIP, "moe_route_sort_static: no device address for the scratch array");
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);  // a lost race stores the same address
  }
  *out = ptr;
  *dev_out = dev;
  return FLUXMI_OK;
}

}  // namespace
}  // namespace fluxmi

extern "C" size_t fluxmi_moe_route_sort_static_max_bytes(void) { return fluxmi::kStaticScratchBytes; }

extern "C" int fluxmi_moe_route_sort_static_init(void) {
  void *ws = nullptr;
  int dev = 0;
  return fluxmi::static_scratch(&ws, &dev);
}

extern "C" int fluxmi_moe_route_sort_static(const int32_t *choosed, int32_t ntokens, int32_t topk,
                                            int32_t nexperts, int32_t *splits, int32_t *offsets,
                                            int32_t *scatter_index, int32_t *gather_index,
                                            int32_t *topk_index, void *stream) {
  using namespace fluxmi;
  const int rc = route_sort_check("moe_route_sort_static", choosed, ntokens, topk, nexperts, scatter_index);
  if (rc != FLUXMI_OK) return rc;
  const size_t need = fluxmi_moe_route_sort_workspace_bytes(ntokens, topk, nexperts);
  FLUXMI_REQUIRE(need <= kStaticScratchBytes, FLUXMI_ERR_WORKSPACE,
                 "moe_route_sort_static: ntokens=%d topk=%d nexperts=%d needs %zu bytes of scratch, the static "
                 "array holds %zu; use fluxmi_moe_route_sort with a workspace",
                 ntokens, topk, nexperts, need, kStaticScratchBytes);
  void *ws = nullptr;
  int dev = 0;
  const int rs = static_scratch(&ws, &dev);
  if (rs != FLUXMI_OK) return rs;
  // Eager calls are chained through an event (created once per device: a host object, no device memory); a call
  // on a capturing stream records nothing outside its graph and is ordered by the graph's own edges.
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  FLUXMI_HIP_CHECK(hipStreamIsCapturing(s, &cap));
  hipEvent_t ev = nullptr;
  if (cap == hipStreamCaptureStatusNone) {
    ev = g_scratch_event[dev].load(std::memory_order_acquire);
    if (ev == nullptr) {
      hipEvent_t fresh = nullptr;
      FLUXMI_HIP_CHECK(hipEventCreateWithFlags(&fresh, hipEventDisableTiming));
      hipEvent_t expected = nullptr;
      if (g_scratch_event[dev].compare_exchange_strong(expected, fresh, std::memory_order_acq_rel)) {
        ev = fresh;
      } else {
        (void)hipEventDestroy(fresh);
        ev = expected;
      }
    } else {
      FLUXMI_HIP_CHECK(hipStreamWaitEvent(s, ev, 0));
    }
  }
  const int rc2 = route_sort_on_workspace(choosed, ntokens, topk, nexperts, splits, offsets, scatter_index, gather_index,
                                          topk_index, ws, stream);
  if (rc2 != FLUXMI_OK) return rc2;
  if (ev != nullptr) FLUXMI_HIP_CHECK(hipEventRecord(ev, s));
  return FLUXMI_OK;
}

extern "C" int fluxmi_moe_gather_index(const int32_t *scatter_index, int32_t nrows, int32_t topk,
                                       int32_t *gather_index, int32_t *topk_index, void *stream) {
  using namespace fluxmi;
  FLUXMI_REQUIRE(nrows >= 0 && topk >= 1, FLUXMI_ERR_INVALID_ARG,
                 "moe_gather_index: bad sizes (nrows=%d, topk=%d)", nrows, topk);
  FLUXMI_REQUIRE(nrows % topk == 0, FLUXMI_ERR_INVALID_ARG,
                 "moe_gather_index: nrows=%d is not a multiple of topk=%d", nrows, topk);
  if (nrows == 0) return FLUXMI_OK;
  FLUXMI_REQUIRE(scatter_index != nullptr && gather_index != nullptr, FLUXMI_ERR_INVALID_ARG,
                 "moe_gather_index: null pointer argument");
  hipLaunchKernelGGL(gather_index_kernel, dim3((nrows + 255) / 256), dim3(256), 0,
                     static_cast<hipStream_t>(stream), scatter_index, nrows, nrows, topk, gather_index,
                     topk_index);
  FLUXMI_HIP_CHECK(hipGetLastError());
  return FLUXMI_OK;
}
