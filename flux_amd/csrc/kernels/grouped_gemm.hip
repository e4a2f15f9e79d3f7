// Grouped GEMM entry point: argument checks, choice between the MFMA kernel and the generic kernel, and
// the generic kernel itself.  The MFMA kernel lives in grouped_gemm_kernel.hpp.
#include "grouped_gemm.hpp"

namespace fluxmi {
namespace {

// ---- generic kernel: any K / N, no alignment demands beyond element size -------------------------
// One thread per output element, a wave covers 64 consecutive columns of one row.  Only used when the
// MFMA kernel's shape requirements do not hold.
__device__ __forceinline__ float e4m3_to_float(uint8_t b) {
  const uint32_t sign = (b & 0x80u) << 24;
  const uint32_t em = b & 0x7fu;
  if (em == 0x7fu) return __uint_as_float(sign | 0x7fc00000u);
  if (em < 8u) return __uint_as_float(sign) + (sign ? -1.f : 1.f) * static_cast<float>(em) * 0x1p-9f;
  return __uint_as_float(sign | ((em + (120u << 3)) << 20));
}

template <int ELT>
__global__ __launch_bounds__(256) void grouped_gemm_generic_kernel(const GemmParams p, const int g) {
  __shared__ int32_t s_row_off[kMaxExperts + 1];
  if (threadIdx.x == 0) {
    int acc = 0;
    for (int e = 0; e < p.nexperts; ++e) {
      s_row_off[e] = acc;
      const int v = p.splits[e];
      acc += v > 0 ? v : 0;
    }
    s_row_off[p.nexperts] = acc;
  }
  __syncthreads();
  const int total_rows = s_row_off[p.nexperts] < p.max_rows ? s_row_off[p.nexperts] : p.max_rows;
  float scalar = p.scalar;
  if (p.scalar_dev) scalar *= p.scalar_dev[0];
  const int ncol_blocks = (p.n + 255) / 256;
  for (int64_t item = blockIdx.x; item < static_cast<int64_t>(total_rows) * ncol_blocks;
       item += gridDim.x) {
    const int r = static_cast<int>(item / ncol_blocks);
    const int n = static_cast<int>(item % ncol_blocks) * 256 + threadIdx.x;
    int e = 0;
    while (r >= s_row_off[e + 1]) ++e;
    if (n >= p.n) continue;
    int64_t arow = r;
    if (p.gather_a) {
      arow = p.gather_a[r];
      if (p.a_rows > 0) arow = arow < 0 ? 0 : (arow >= p.a_rows ? p.a_rows - 1 : arow);
    }
    const uint8_t *ap = p.a + arow * p.k * ELT;
    const uint8_t *bp = p.b[g] + (static_cast<int64_t>(e) * p.n + n) * p.k * ELT;
    float acc = 0.f, total = 0.f;
    const int kblocks = p.k / 128;
    for (int kk = 0; kk < p.k; ++kk) {
      float av, bv;
      if (ELT == 2) {
        const uint16_t ab = reinterpret_cast<const uint16_t *>(ap)[kk], bb = reinterpret_cast<const uint16_t *>(bp)[kk];
        av = p.half_is_f16 ? f16_bits_to_float(ab) : bf16_bits_to_float(ab);
        bv = p.half_is_f16 ? f16_bits_to_float(bb) : bf16_bits_to_float(bb);
      } else {
        av = e4m3_to_float(ap[kk]);
        bv = e4m3_to_float(bp[kk]);
      }
      acc = fmaf(av, bv, acc);
      if (p.a_scale != nullptr && (kk & 127) == 127) {  // end of a scale block of K: promote
        const int kb = kk >> 7, nb = n >> 7, nblocks = (p.n + 127) >> 7;
        const float as = p.a_scale_layout == FLUXMI_ASCALE_BLOCK128
                             ? p.a_scale[((arow >> 7) * kblocks + kb) * 128 + (arow & 127)]
                             : p.a_scale[static_cast<int64_t>(s_row_off[e]) * kblocks +
                                         static_cast<int64_t>(kb) * (s_row_off[e + 1] - s_row_off[e]) + (r - s_row_off[e])];
        const float bs = p.b_scale_layout == FLUXMI_BSCALE_N_K
                             ? p.b_scale[(static_cast<int64_t>(e) * nblocks + nb) * kblocks + kb]
                             : p.b_scale_layout == FLUXMI_BSCALE_K_N
                                   ? p.b_scale[(static_cast<int64_t>(e) * kblocks + kb) * nblocks + nb]
                                   : p.b_scale[((static_cast<int64_t>(e) * nblocks + nb) * kblocks + kb) * 128 + (n & 127)];
        total = fmaf(acc, as * bs, total);
        acc = 0.f;
      }
    }
    if (p.a_scale != nullptr) acc = total;
    float v = acc * scalar * (p.alpha[g] ? p.alpha[g][e] : 1.f) * (p.row_scale ? p.row_scale[r] : 1.f);
    if (p.col_scale) v *= p.col_scale[static_cast<int64_t>(e) * p.n + n];
    int64_t drow = r;
    if (p.scatter_d) {
      drow = p.scatter_d[r];
      if (drow < 0 || drow >= p.d_rows) continue;
    }
    if (p.accumulate) unsafeAtomicAdd(static_cast<float *>(p.d[g]) + drow * p.n + n, v);
    else if (p.d_fp32) static_cast<float *>(p.d[g])[drow * p.n + n] = v;
    else static_cast<uint16_t *>(p.d[g])[drow * p.n + n] = p.half_is_f16 ? float_to_f16_bits(v) : float_to_bf16_bits(v);
  }
}

// Shapes the MFMA kernel takes: rows of K a multiple of 16 bytes (K % 8 == 0 for bf16, K % 16 == 0 for fp8),
// N a multiple of 4, aligned pointers, and operands its 32-bit buffer offsets can span (a gathered A as a
// whole, which needs its extent a_rows; 256 rows of an ungathered A; one expert's weights).  Everything else
// runs the generic kernel.
bool mfma_path_ok(const fluxmi_grouped_gemm_args *a, const void *b, const void *d, bool d_is_fp32) {
  const int elt = a->dtype == FLUXMI_FP8_E4M3 ? 1 : 2;
  const int64_t kbytes = static_cast<int64_t>(a->k) * elt;
  const int64_t span = 0xffffffffll;
  const bool a_fits = a->gather_a ? (a->a_rows > 0 && a->a_rows * kbytes <= span) : BM * kbytes <= span;
  return kbytes % 16 == 0 && kbytes >= 16 && a->n % 4 == 0 && aligned16(a->a) &&
         aligned16(b) && (reinterpret_cast<uintptr_t>(d) & (d_is_fp32 ? 15u : 7u)) == 0 &&
         (a->col_scale == nullptr || aligned16(a->col_scale)) && a_fits && a->n * kbytes <= span;
}

}  // namespace
}  // namespace fluxmi

extern "C" size_t fluxmi_grouped_gemm_workspace_bytes(const fluxmi_grouped_gemm_args *) { return 0; }

namespace fluxmi {
namespace {

// dry_run: check the arguments and report which kernel would run (1 MFMA, 0 generic) without launching.
// accumulate_rows > 0: D is fp32 with that many rows and results are added to it atomically.
struct BlockScales {
  const float *a_scale = nullptr, *b_scale = nullptr;
  int32_t a_layout = 0, b_layout = 0;
};

int run_grouped_gemm(const fluxmi_grouped_gemm_args *args, int ngroups, const void *const *b, void *const *d,
                     const float *const *alpha, void *stream, bool dry_run = false, int32_t accumulate_rows = 0,
                     const BlockScales *bs = nullptr) {
  FLUXMI_REQUIRE(args != nullptr, FLUXMI_ERR_INVALID_ARG, "grouped_gemm: null args");
  FLUXMI_REQUIRE(args->dtype == FLUXMI_BF16 || args->dtype == FLUXMI_FP8_E4M3 || args->dtype == FLUXMI_FP16, FLUXMI_ERR_INVALID_ARG,
                 "grouped_gemm: unknown dtype %d", args->dtype);
  FLUXMI_REQUIRE(args->d_fp32 == 0 || args->d_fp32 == 1, FLUXMI_ERR_INVALID_ARG,
                 "grouped_gemm: d_fp32 must be 0 or 1");
  FLUXMI_REQUIRE(args->a_rows >= 0, FLUXMI_ERR_INVALID_ARG, "grouped_gemm: negative a_rows");
  FLUXMI_REQUIRE(args->reserved == 0, FLUXMI_ERR_INVALID_ARG, "grouped_gemm: reserved must be 0, got %d",
                 args->reserved);
  FLUXMI_REQUIRE(args->nexperts >= 1 && args->nexperts <= kMaxExperts, FLUXMI_ERR_UNSUPPORTED,
                 "grouped_gemm: nexperts=%d outside [1,%d]", args->nexperts, kMaxExperts);
  FLUXMI_REQUIRE(args->max_rows >= 0 && args->n >= 0 && args->k >= 0, FLUXMI_ERR_INVALID_ARG,
                 "grouped_gemm: negative size (max_rows=%d, n=%d, k=%d)", args->max_rows, args->n,
                 args->k);
  FLUXMI_REQUIRE(ngroups >= 1 && ngroups <= kMaxWeightGroups, FLUXMI_ERR_UNSUPPORTED,
                 "grouped_gemm: ngroups=%d outside [1,%d]", ngroups, kMaxWeightGroups);
  if (args->max_rows == 0 || args->n == 0) return dry_run ? 1 : FLUXMI_OK;
  FLUXMI_REQUIRE(args->k >= 1, FLUXMI_ERR_UNSUPPORTED, "grouped_gemm: k must be positive");
  FLUXMI_REQUIRE(args->a && args->splits && b && d, FLUXMI_ERR_INVALID_ARG, "grouped_gemm: null a / b / d / splits");

  GemmParams p;
  bool mfma = true;
  for (int g = 0; g < kMaxWeightGroups; ++g) {
    const int src = g < ngroups ? g : 0;
    FLUXMI_REQUIRE(b[src] && d[src], FLUXMI_ERR_INVALID_ARG, "grouped_gemm: null b / d of weight group %d", src);
    p.b[g] = static_cast<const uint8_t *>(b[src]);
    p.d[g] = d[src];
    p.alpha[g] = alpha ? alpha[src] : nullptr;
    mfma = mfma && mfma_path_ok(args, b[src], d[src], accumulate_rows > 0 || args->d_fp32 != 0);
  }
  // The tile schedule numbers the column tiles of all groups with one int.
  mfma = mfma && (static_cast<int64_t>(args->n) + BN) * ngroups < (1ll << 30);
  p.a = static_cast<const uint8_t *>(args->a);
  p.splits = args->splits;
  p.gather_a = args->gather_a;
  p.scatter_d = args->scatter_d;
  p.row_scale = args->row_scale;
  p.col_scale = args->col_scale;
  p.scalar_dev = args->scalar_scale_dev;
  p.scalar = args->scalar_scale;
  p.nexperts = args->nexperts;
  p.max_rows = args->max_rows;
  p.a_rows = args->a_rows;
  p.n = args->n;
  p.k = args->k;
  p.d_fp32 = accumulate_rows > 0 ? 1 : args->d_fp32;
  p.accumulate = accumulate_rows > 0 ? 1 : 0;
  p.d_rows = accumulate_rows > 0 ? accumulate_rows : args->max_rows;
  p.ngroups = ngroups;
  p.half_is_f16 = args->dtype == FLUXMI_FP16 ? 1 : 0;
  p.a_scale = bs ? bs->a_scale : nullptr;
  p.b_scale = bs ? bs->b_scale : nullptr;
  p.a_scale_layout = bs ? bs->a_layout : 0;
  p.b_scale_layout = bs ? bs->b_layout : 0;
  if (bs != nullptr) {
    FLUXMI_REQUIRE(args->dtype == FLUXMI_FP8_E4M3, FLUXMI_ERR_UNSUPPORTED, "grouped_gemm_blockscale: dtype must be fp8 e4m3");
    FLUXMI_REQUIRE(args->k % 128 == 0, FLUXMI_ERR_UNSUPPORTED, "grouped_gemm_blockscale: K=%d is not a multiple of 128", args->k);
    FLUXMI_REQUIRE(bs->a_scale != nullptr && bs->b_scale != nullptr, FLUXMI_ERR_INVALID_ARG,
                   "grouped_gemm_blockscale: null a_scale / b_scale");
    FLUXMI_REQUIRE((bs->a_layout == FLUXMI_ASCALE_BLOCK128 || bs->a_layout == FLUXMI_ASCALE_EXPERT_K_M) &&
                       (bs->b_layout == FLUXMI_BSCALE_N_K || bs->b_layout == FLUXMI_BSCALE_K_N ||
                        bs->b_layout == FLUXMI_BSCALE_COL_N_K),
                   FLUXMI_ERR_INVALID_ARG, "grouped_gemm_blockscale: unknown scale layout (%d, %d)", bs->a_layout, bs->b_layout);
    FLUXMI_REQUIRE(!(bs->a_layout == FLUXMI_ASCALE_EXPERT_K_M && args->gather_a != nullptr), FLUXMI_ERR_INVALID_ARG,
                   "grouped_gemm_blockscale: per-expert a_scale segments cannot be combined with gather_a");
    FLUXMI_REQUIRE(ngroups == 1, FLUXMI_ERR_UNSUPPORTED, "grouped_gemm_blockscale: one weight tensor per launch");
    if (bs->b_layout == FLUXMI_BSCALE_COL_N_K) mfma = false;  // per-column weight scales: the generic kernel only
    // a_scale is addressed with 32-bit byte offsets
    const int64_t srows = args->gather_a ? args->a_rows : args->max_rows;
    mfma = mfma && ((srows + 127) / 128 * 128) * (args->k / 128) * 4 < (int64_t{1} << 32) &&
           (reinterpret_cast<uintptr_t>(bs->a_scale) & 3u) == 0;
  }
  FLUXMI_REQUIRE(args->raster_rows >= 0 && args->raster_rows <= 1024, FLUXMI_ERR_INVALID_ARG,
                 "grouped_gemm: raster_rows=%d outside [0,1024]", args->raster_rows);
  FLUXMI_REQUIRE(args->cu_margin >= 0, FLUXMI_ERR_INVALID_ARG, "grouped_gemm: negative cu_margin");
  FLUXMI_REQUIRE((args->sched_flags & ~(FLUXMI_SCHED_WHOLE_TAIL_TILES | FLUXMI_SCHED_NO_HALF_TILES |
                                        FLUXMI_SCHED_NO_SKINNY_TAIL | FLUXMI_SCHED_FORCE_SKINNY_TAIL | FLUXMI_SCHED_HALF_LINE_FILLS |
                                        FLUXMI_SCHED_WHOLE_LINE_FILLS)) == 0,
                 FLUXMI_ERR_INVALID_ARG, "grouped_gemm: unknown sched_flags 0x%x", args->sched_flags);
  FLUXMI_REQUIRE((args->sched_flags & FLUXMI_SCHED_HALF_LINE_FILLS) == 0 || (args->sched_flags & FLUXMI_SCHED_WHOLE_LINE_FILLS) == 0,
                 FLUXMI_ERR_INVALID_ARG, "grouped_gemm: sched_flags ask for half-line and whole-line fills at once");
  // fp32 outputs beyond half a GB go out non-temporally (measured on a 805 MB intermediate: the GEMM 5 % faster,
  // the reduce that reads it unchanged; at 268 MB the GEMM is unchanged and the reduce 10 % slower).
  p.nt_stores = (args->d_fp32 != 0 && accumulate_rows == 0 && static_cast<int64_t>(args->max_rows) * args->n * 4 > (int64_t{512} << 20)) ? 1 : 0;
  p.raster_rows = args->raster_rows > 0 ? args->raster_rows : 8;
  p.sched_flags = args->sched_flags;

  if (dry_run) return mfma ? 1 : 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  int cus = fluxmi_device_cu_count();
  FLUXMI_REQUIRE(cus > 0, FLUXMI_ERR_HIP, "grouped_gemm: cannot query the device");
  // CUs left to other work of the caller (Flux's sm_margin): the persistent kernel launches fewer workgroups.
  cus = cus - args->cu_margin > 1 ? cus - args->cu_margin : 1;

  if (mfma) {
    // Upper bound of the tile count: never launch more workgroups than tiles.
    const int64_t tiles_n = (args->n + BN - 1) / BN * ngroups;
    const int64_t max_tiles = (static_cast<int64_t>(args->max_rows) / BM + args->nexperts) * tiles_n;
    const int grid = static_cast<int>(max_tiles < cus ? max_tiles : cus);
    // Form of the ring fills.  Whole 128-byte lines cost the memory pipeline less per byte and need one barrier per
    // pair of k-steps, but a pair's 64 KiB stay in LDS for both of its steps, so fewer fills are in flight: faster
    // (2-5 %) where the compute units that share operand panels run in step (uniform row counts) or K is long, slower
    // (up to 7 %) on ragged row counts at short K, where single units run ahead of the others and every one of their
    // fills misses L2.  Default: whole lines for rows that are not gathered and hold at least 16 KiB of K (measured on
    // 8 ragged experts at K = 14336 bf16: -1.2 ... -2.5 %), half lines otherwise (a single-expert rule was tried: the
    // dense bf16 GEMM 4096 x 12288 x 6144 gains under 1 %, the dense fp8 GEMMs 32768 x 7168 x 2048 lose 3-6 %); the flags force either, and `profiling()`
    // of the layer ops times both on the caller's own row counts.
    const int64_t kbytes = static_cast<int64_t>(args->k) * (args->dtype == FLUXMI_FP8_E4M3 ? 1 : 2);
    const bool lines = (args->sched_flags & FLUXMI_SCHED_WHOLE_LINE_FILLS) != 0 ||
                       ((args->sched_flags & FLUXMI_SCHED_HALF_LINE_FILLS) == 0 && args->gather_a == nullptr && kbytes >= 16384);
    const int rc = bs != nullptr ? launch_grouped_gemm_fp8_blockscale(p, grid, s)
                   : args->dtype == FLUXMI_BF16 ? (lines ? launch_grouped_gemm_bf16_lines(p, grid, s) : launch_grouped_gemm_bf16(p, grid, s))
                   : args->dtype == FLUXMI_FP16 ? launch_grouped_gemm_f16(p, grid, s)  // the half-line form only
                                                : (lines ? launch_grouped_gemm_fp8_lines(p, grid, s) : launch_grouped_gemm_fp8(p, grid, s));
    if (rc != FLUXMI_OK) return rc;
  } else {
    const int grid = cus * 8;
    for (int g = 0; g < ngroups; ++g) {
      if (args->dtype != FLUXMI_FP8_E4M3)
        hipLaunchKernelGGL(grouped_gemm_generic_kernel<2>, dim3(grid), dim3(256), 0, s, p, g);
      else
        hipLaunchKernelGGL(grouped_gemm_generic_kernel<1>, dim3(grid), dim3(256), 0, s, p, g);
    }
  }
  FLUXMI_HIP_CHECK(hipGetLastError());
  return FLUXMI_OK;
}

}  // namespace
}  // namespace fluxmi

extern "C" int fluxmi_grouped_gemm(const fluxmi_grouped_gemm_args *args, void *, size_t, void *stream) {
  FLUXMI_REQUIRE(args != nullptr, FLUXMI_ERR_INVALID_ARG, "grouped_gemm: null args");
  const void *b = args->b;
  void *d = args->d;
  const float *alpha = args->alpha;
  return fluxmi::run_grouped_gemm(args, 1, &b, &d, &alpha, stream);
}

namespace fluxmi {
namespace {

typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

// 16-byte units of fp32 accumulators: cleared before the accumulating GEMM (a fill kernel, not a memset node,
// so that the sequence can be captured in a HIP graph) and rounded to bf16 after it.
__global__ __launch_bounds__(256) void zero_f32x4_kernel(float4 *__restrict__ dst, int64_t nvec) {
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < nvec; i += static_cast<int64_t>(gridDim.x) * 256)
    dst[i] = make_float4(0.f, 0.f, 0.f, 0.f);
}

template <bool F16>
__global__ __launch_bounds__(256) void cast_f32x4_half_kernel(const float4 *__restrict__ src, u32x2_t *__restrict__ dst,
                                                              int64_t nvec) {
  auto cvt = [](float f) { return static_cast<uint32_t>(F16 ? float_to_f16_bits(f) : float_to_bf16_bits(f)); };
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < nvec; i += static_cast<int64_t>(gridDim.x) * 256) {
    const float4 v = src[i];
    u32x2_t o;
    o[0] = cvt(v.x) | (cvt(v.y) << 16);
    o[1] = cvt(v.z) | (cvt(v.w) << 16);
    __builtin_nontemporal_store(o, dst + i);
  }
}

}  // namespace
}  // namespace fluxmi

extern "C" size_t fluxmi_grouped_gemm_topk_reduce_workspace_bytes(int32_t ntokens, int32_t n) {
  if (ntokens < 0 || n < 0) return 0;
  return static_cast<size_t>(ntokens) * static_cast<size_t>(n) * sizeof(float);
}

extern "C" int fluxmi_grouped_gemm_topk_reduce(const fluxmi_grouped_gemm_args *args, const int32_t *token_of_row,
                                               int32_t ntokens, void *out, void *workspace, size_t workspace_bytes,
                                               void *stream) {
  using namespace fluxmi;
  FLUXMI_REQUIRE(args != nullptr, FLUXMI_ERR_INVALID_ARG, "grouped_gemm_topk_reduce: null args");
  FLUXMI_REQUIRE(ntokens >= 0 && args->n >= 0, FLUXMI_ERR_INVALID_ARG, "grouped_gemm_topk_reduce: negative size");
  FLUXMI_REQUIRE(args->scatter_d == nullptr, FLUXMI_ERR_INVALID_ARG,
                 "grouped_gemm_topk_reduce: scatter_d must be NULL (token_of_row takes its place)");
  if (ntokens == 0 || args->n == 0) return FLUXMI_OK;
  FLUXMI_REQUIRE(token_of_row != nullptr && out != nullptr, FLUXMI_ERR_INVALID_ARG,
                 "grouped_gemm_topk_reduce: null token_of_row / out");
  FLUXMI_REQUIRE(args->n % 4 == 0 && (reinterpret_cast<uintptr_t>(out) & 7u) == 0, FLUXMI_ERR_UNSUPPORTED,
                 "grouped_gemm_topk_reduce: n must be a multiple of 4 and out 8-byte aligned");
  const size_t need = fluxmi_grouped_gemm_topk_reduce_workspace_bytes(ntokens, args->n);
  FLUXMI_REQUIRE(workspace != nullptr && workspace_bytes >= need && aligned16(workspace), FLUXMI_ERR_WORKSPACE,
                 "grouped_gemm_topk_reduce: a 16-byte aligned workspace of %zu bytes is needed, %zu given", need,
                 workspace_bytes);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t nvec = static_cast<int64_t>(ntokens) * args->n / 4;
  int cus = fluxmi_device_cu_count();
  FLUXMI_REQUIRE(cus > 0, FLUXMI_ERR_HIP, "grouped_gemm_topk_reduce: cannot query the device");
  const int64_t want = (nvec + 255) / 256;
  const unsigned grid = static_cast<unsigned>(want < static_cast<int64_t>(cus) * 16 ? want : static_cast<int64_t>(cus) * 16);
  hipLaunchKernelGGL(zero_f32x4_kernel, dim3(grid), dim3(256), 0, s, static_cast<float4 *>(workspace), nvec);
  fluxmi_grouped_gemm_args a = *args;
  a.scatter_d = token_of_row;
  const void *b = a.b;
  void *d = workspace;
  const float *alpha = a.alpha;
  const int rc = run_grouped_gemm(&a, 1, &b, &d, &alpha, stream, false, ntokens);
  if (rc != FLUXMI_OK) return rc;
  if (args->dtype == FLUXMI_FP16)
    hipLaunchKernelGGL(cast_f32x4_half_kernel<true>, dim3(grid), dim3(256), 0, s, static_cast<const float4 *>(workspace),
                       static_cast<u32x2_t *>(out), nvec);
  else
    hipLaunchKernelGGL(cast_f32x4_half_kernel<false>, dim3(grid), dim3(256), 0, s, static_cast<const float4 *>(workspace),
                       static_cast<u32x2_t *>(out), nvec);
  FLUXMI_HIP_CHECK(hipGetLastError());
  return FLUXMI_OK;
}

extern "C" int fluxmi_grouped_gemm_blockscale(const fluxmi_grouped_gemm_args *args, const float *a_scale,
                                              int32_t a_scale_layout, const float *b_scale, int32_t b_scale_layout,
                                              void *stream) {
  FLUXMI_REQUIRE(args != nullptr, FLUXMI_ERR_INVALID_ARG, "grouped_gemm_blockscale: null args");
  fluxmi::BlockScales bs;
  bs.a_scale = a_scale;
  bs.b_scale = b_scale;
  bs.a_layout = a_scale_layout;
  bs.b_layout = b_scale_layout;
  const void *b = args->b;
  void *d = args->d;
  const float *alpha = args->alpha;
  return fluxmi::run_grouped_gemm(args, 1, &b, &d, &alpha, stream, false, 0, &bs);
}

extern "C" int fluxmi_grouped_gemm_kernel_kind(const fluxmi_grouped_gemm_args *args) {
  FLUXMI_REQUIRE(args != nullptr, FLUXMI_ERR_INVALID_ARG, "grouped_gemm: null args");
  const void *b = args->b;
  void *d = args->d;
  const float *alpha = args->alpha;
  return fluxmi::run_grouped_gemm(args, 1, &b, &d, &alpha, nullptr, /*dry_run=*/true);
}

extern "C" int fluxmi_grouped_gemm_multi(const fluxmi_grouped_gemm_args *args, int32_t ngroups, const void *const *b,
                                         void *const *d, const float *const *alpha, void *, size_t, void *stream) {
  return fluxmi::run_grouped_gemm(args, ngroups, b, d, alpha, stream);
}
