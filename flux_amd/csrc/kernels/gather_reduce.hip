// Top-k (weighted) gather-reduce: out[t,:] = bf16(scale * sum_g sum_j w[r_j] * in_g[r_j,:]).
//
// HBM-streaming kernel.  One workgroup owns one token row (or a column slab of it); every lane moves
// 16-byte vectors (8 bf16), so a wave touches 1 KiB of contiguous row per instruction.  All top-k
// source rows of a token are fetched before the first add so that topk*ngroups loads are in flight per
// lane.  Source rows are read exactly once in the whole launch, hence the non-temporal loads.
#include "common.hpp"

namespace fluxmi {
namespace {

constexpr int kMaxGroups = 4;
constexpr int kMaxThreads = 512;
// Inputs up to this size are read with ordinary loads: small enough to sit in the 256 MiB Infinity Cache
// whole, which non-temporal loads do not use as well.  Larger inputs are read non-temporally: they stream
// from HBM, also right after the grouped GEMM that wrote them (measured inside a layer: 268 MB of fp32
// rows 5.6 TB/s with ordinary loads, 6.4 TB/s non-temporally; 134 MB the same either way).
constexpr size_t kPlainLoadMaxBytes = size_t{128} << 20;

struct GroupPtrs {
  const void *p[kMaxGroups];
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Eight consecutive elements of a source row as loaded: one 16-byte vector of bf16, or two of fp32.
template <bool IN_F32>
struct Vec8 {
  u32x4 v[IN_F32 ? 2 : 1];
};

template <bool NT>
__device__ __forceinline__ u32x4 load16(const u32x4 *src) {
  if constexpr (NT) return __builtin_nontemporal_load(src);
  else return *src;
}

template <bool IN_F32, bool NT>
__device__ __forceinline__ Vec8<IN_F32> load8(const void *base, size_t row, size_t row_vecs, int v) {
  Vec8<IN_F32> r;
  if constexpr (IN_F32) {
    const u32x4 *src = reinterpret_cast<const u32x4 *>(base) + (row * row_vecs + v) * 2;
    r.v[0] = load16<NT>(src);
    r.v[1] = load16<NT>(src + 1);
  } else {
    r.v[0] = load16<NT>(reinterpret_cast<const u32x4 *>(base) + row * row_vecs + v);
  }
  return r;
}

template <bool IN_F32>
__device__ __forceinline__ Vec8<IN_F32> zero8() {
  Vec8<IN_F32> r;
#pragma unroll
  for (int i = 0; i < (IN_F32 ? 2 : 1); ++i) r.v[i] = u32x4{0u, 0u, 0u, 0u};
  return r;
}

// F16: 16-bit inputs are fp16 instead of bf16; fp32 inputs ignore it.
template <bool F16>
__device__ __forceinline__ void accumulate8(float (&acc)[8], const Vec8<true> &x, const float w) {
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = fmaf(w, __uint_as_float(x.v[i >> 2][i & 3]), acc[i]);
}

template <bool F16>
__device__ __forceinline__ void accumulate8(float (&acc)[8], const Vec8<false> &x, const float w) {
  const u32x4 v = x.v[0];
  if constexpr (F16) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t u = v[i];
      acc[2 * i] = fmaf(w, f16_bits_to_float(static_cast<uint16_t>(u & 0xffffu)), acc[2 * i]);
      acc[2 * i + 1] = fmaf(w, f16_bits_to_float(static_cast<uint16_t>(u >> 16)), acc[2 * i + 1]);
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t u = v[i];
    acc[2 * i] = fmaf(w, __uint_as_float(u << 16), acc[2 * i]);
    acc[2 * i + 1] = fmaf(w, __uint_as_float(u & 0xffff0000u), acc[2 * i + 1]);
  }
}

// A routing entry names a source row only inside [0, nrows): negative entries mark dropped pairs, and an
// entry at or past the end of the input must never be dereferenced.
__device__ __forceinline__ bool row_in_range(int32_t r, int32_t nrows) {
  return static_cast<uint32_t>(r) < static_cast<uint32_t>(nrows);
}

// Two results to the packed 16-bit output type: bf16, or fp16.
template <bool F16>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  if constexpr (F16) return static_cast<uint32_t>(float_to_f16_bits(lo)) | (static_cast<uint32_t>(float_to_f16_bits(hi)) << 16);
  return static_cast<uint32_t>(float_to_bf16_bits(lo)) | (static_cast<uint32_t>(float_to_bf16_bits(hi)) << 16);
}

// TOPK > 0: compile-time top-k (loads fully unrolled).  TOPK == 0: run-time top-k.
// NT: non-temporal source loads.  The choice is made once per launch and hoisted out of the load
// sequence, so that no control flow sits between the loads of one output vector.
template <int TOPK, int NGROUPS, bool WEIGHTED, bool IN_F32, bool NT, bool F16>
__device__ __forceinline__ void topk_gather_reduce_body(
    const GroupPtrs &in, const int32_t *__restrict__ routing_idx, const float *__restrict__ row_weight,
    float scale, int32_t topk_rt, int32_t nvec, int32_t nrows, uint16_t *__restrict__ out) {
  const int t = blockIdx.x;
  const int topk = TOPK > 0 ? TOPK : topk_rt;
  const size_t row_vecs = static_cast<size_t>(nvec);
  const int nthreads = blockDim.x;
  if constexpr (IN_F32 && TOPK > 0) {
    // fp32 rows: a lane takes the 16-byte units q and q + nthreads of a pass (not two adjacent ones), so that
    // every load instruction of a wave covers 1 KiB of contiguous row, as in the bf16 case.
    const int nq = 2 * nvec;  // 16-byte units (4 elements) per source row
    for (int q0 = blockIdx.y * 2 * nthreads; q0 < nq; q0 += gridDim.y * 2 * nthreads) {
      const int qa = q0 + threadIdx.x, qb = qa + nthreads;
      const bool oka = qa < nq, okb = qb < nq;
      u32x4 va[NGROUPS][TOPK], vb[NGROUPS][TOPK];
      float w[TOPK];
#pragma unroll
      for (int j = 0; j < TOPK; ++j) {
        const int32_t r = routing_idx[static_cast<size_t>(t) * TOPK + j];
        const bool live = row_in_range(r, nrows);
        w[j] = 0.f;
        if (live) w[j] = WEIGHTED ? row_weight[r] : 1.f;
#pragma unroll
        for (int g = 0; g < NGROUPS; ++g) {
          va[g][j] = u32x4{0u, 0u, 0u, 0u};
          vb[g][j] = u32x4{0u, 0u, 0u, 0u};
          const u32x4 *src = reinterpret_cast<const u32x4 *>(in.p[g]) + static_cast<size_t>(live ? r : 0) * nq;
          if (live && oka) va[g][j] = load16<NT>(src + qa);
          if (live && okb) vb[g][j] = load16<NT>(src + qb);
        }
      }
      float a[4] = {0.f, 0.f, 0.f, 0.f}, b[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int g = 0; g < NGROUPS; ++g) {
#pragma unroll
        for (int j = 0; j < TOPK; ++j) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            a[i] = fmaf(w[j], __uint_as_float(va[g][j][i]), a[i]);
            b[i] = fmaf(w[j], __uint_as_float(vb[g][j][i]), b[i]);
          }
        }
      }
      typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
      u32x2 *dst = reinterpret_cast<u32x2 *>(out) + static_cast<size_t>(t) * nq;
      if (oka) {
        u32x2 o;
        o[0] = pack2<F16>(a[0] * scale, a[1] * scale);
        o[1] = pack2<F16>(a[2] * scale, a[3] * scale);
        __builtin_nontemporal_store(o, dst + qa);
      }
      if (okb) {
        u32x2 o;
        o[0] = pack2<F16>(b[0] * scale, b[1] * scale);
        o[1] = pack2<F16>(b[2] * scale, b[3] * scale);
        __builtin_nontemporal_store(o, dst + qb);
      }
    }
    return;
  }
  for (int v = blockIdx.y * nthreads + threadIdx.x; v < nvec; v += gridDim.y * nthreads) {
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if constexpr (TOPK > 0) {
      Vec8<IN_F32> vals[NGROUPS][TOPK];
      float w[TOPK];
#pragma unroll
      for (int j = 0; j < TOPK; ++j) {
        const int32_t r = routing_idx[static_cast<size_t>(t) * TOPK + j];
        const bool live = row_in_range(r, nrows);
        w[j] = 0.f;
        if (live) w[j] = WEIGHTED ? row_weight[r] : 1.f;
#pragma unroll
        for (int g = 0; g < NGROUPS; ++g) {
          vals[g][j] = zero8<IN_F32>();
          // r is wave-uniform: a skipped (dropped or out-of-range) row costs no traffic
          if (live) vals[g][j] = load8<IN_F32, NT>(in.p[g], static_cast<size_t>(r), row_vecs, v);
        }
      }
#pragma unroll
      for (int g = 0; g < NGROUPS; ++g) {
#pragma unroll
        for (int j = 0; j < TOPK; ++j) accumulate8<F16>(acc, vals[g][j], w[j]);
      }
    } else {
      for (int g = 0; g < NGROUPS; ++g) {
        for (int j = 0; j < topk; ++j) {
          const int32_t r = routing_idx[static_cast<size_t>(t) * topk + j];
          if (!row_in_range(r, nrows)) continue;
          const float w = WEIGHTED ? row_weight[r] : 1.f;
          accumulate8<F16>(acc, load8<IN_F32, NT>(in.p[g], static_cast<size_t>(r), row_vecs, v), w);
        }
      }
    }
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = pack2<F16>(acc[2 * i] * scale, acc[2 * i + 1] * scale);
    u32x4 *dst = reinterpret_cast<u32x4 *>(out) + static_cast<size_t>(t) * row_vecs + v;
    __builtin_nontemporal_store(o, dst);
  }
}

template <int TOPK, int NGROUPS, bool WEIGHTED, bool IN_F32, bool F16>
__global__ __launch_bounds__(kMaxThreads) void topk_gather_reduce_kernel(
    GroupPtrs in, const int32_t *__restrict__ routing_idx, const float *__restrict__ row_weight,
    float scale, int32_t topk_rt, int32_t nvec /* n / 8 */, int32_t nrows, int32_t nt_loads,
    uint16_t *__restrict__ out) {
  if (nt_loads)
    topk_gather_reduce_body<TOPK, NGROUPS, WEIGHTED, IN_F32, true, F16>(in, routing_idx, row_weight, scale, topk_rt,
                                                                        nvec, nrows, out);
  else
    topk_gather_reduce_body<TOPK, NGROUPS, WEIGHTED, IN_F32, false, F16>(in, routing_idx, row_weight, scale, topk_rt,
                                                                         nvec, nrows, out);
}

// F16 (fp16 inputs and / or output) exists for the run-time top-k form only: the unrolled forms are the bf16 path's.
template <int TOPK, int NGROUPS, bool F16 = false>
void launch(bool weighted, bool in_f32, dim3 grid, int threads, int nt, hipStream_t s, const GroupPtrs &in,
            const int32_t *idx, const float *w, float scale, int32_t topk, int32_t nvec, int32_t nrows, uint16_t *out) {
#define FLUXMI_GR_LAUNCH(W, F)                                                                            \
  hipLaunchKernelGGL((topk_gather_reduce_kernel<TOPK, NGROUPS, W, F, F16>), grid, dim3(threads), 0, s, in, \
                     idx, w, scale, topk, nvec, nrows, nt, out)
  if (weighted) {
    if (in_f32) FLUXMI_GR_LAUNCH(true, true);
    else FLUXMI_GR_LAUNCH(true, false);
  } else {
    if (in_f32) FLUXMI_GR_LAUNCH(false, true);
    else FLUXMI_GR_LAUNCH(false, false);
  }
#undef FLUXMI_GR_LAUNCH
}

template <int NGROUPS>
void dispatch_topk(bool weighted, bool in_f32, dim3 grid, int threads, int nt, hipStream_t s, const GroupPtrs &in, const int32_t *idx,
                   const float *w, float scale, int32_t topk, int32_t nvec, int32_t nrows, uint16_t *out, bool f16) {
  if (f16) {
    launch<0, NGROUPS, true>(weighted, in_f32, grid, threads, nt, s, in, idx, w, scale, topk, nvec, nrows, out);
    return;
  }
  switch (topk) {
    case 1: launch<1, NGROUPS>(weighted, in_f32, grid, threads, nt, s, in, idx, w, scale, topk, nvec, nrows, out); break;
    case 2: launch<2, NGROUPS>(weighted, in_f32, grid, threads, nt, s, in, idx, w, scale, topk, nvec, nrows, out); break;
    case 4: launch<4, NGROUPS>(weighted, in_f32, grid, threads, nt, s, in, idx, w, scale, topk, nvec, nrows, out); break;
    case 6: launch<6, NGROUPS>(weighted, in_f32, grid, threads, nt, s, in, idx, w, scale, topk, nvec, nrows, out); break;
    case 8: launch<8, NGROUPS>(weighted, in_f32, grid, threads, nt, s, in, idx, w, scale, topk, nvec, nrows, out); break;
    default: launch<0, NGROUPS>(weighted, in_f32, grid, threads, nt, s, in, idx, w, scale, topk, nvec, nrows, out); break;
  }
}

}  // namespace
}  // namespace fluxmi

extern "C" int fluxmi_topk_gather_reduce(const void *const *in, int32_t ngroups, int32_t io_format,
                                         const int32_t *routing_idx, const float *row_weight,
                                         float scale, int32_t ntokens, int32_t topk, int32_t n,
                                         void *out, void *stream) {
  using namespace fluxmi;
  FLUXMI_REQUIRE(in != nullptr && routing_idx != nullptr && out != nullptr, FLUXMI_ERR_INVALID_ARG,
                 "topk_gather_reduce: null pointer argument");
  FLUXMI_REQUIRE(io_format >= 0 && io_format <= 3, FLUXMI_ERR_INVALID_ARG,
                 "topk_gather_reduce: io_format=%d outside [0,3]", io_format);
  const int32_t in_fp32 = io_format & 1;
  const bool half_f16 = (io_format & 2) != 0;
  FLUXMI_REQUIRE(ngroups >= 1 && ngroups <= kMaxGroups, FLUXMI_ERR_UNSUPPORTED,
                 "topk_gather_reduce: ngroups=%d outside [1,%d]", ngroups, kMaxGroups);
  FLUXMI_REQUIRE(topk >= 1 && topk <= 64, FLUXMI_ERR_UNSUPPORTED,
                 "topk_gather_reduce: topk=%d outside [1,64]", topk);
  FLUXMI_REQUIRE(ntokens >= 0 && n >= 0, FLUXMI_ERR_INVALID_ARG,
                 "topk_gather_reduce: negative size (ntokens=%d, n=%d)", ntokens, n);
  FLUXMI_REQUIRE(n % 8 == 0, FLUXMI_ERR_UNSUPPORTED, "topk_gather_reduce: n=%d is not a multiple of 8",
                 n);
  GroupPtrs gp{};
  for (int g = 0; g < ngroups; ++g) {
    FLUXMI_REQUIRE(in[g] != nullptr && aligned16(in[g]), FLUXMI_ERR_INVALID_ARG,
                   "topk_gather_reduce: input group %d is null or not 16-byte aligned", g);
    gp.p[g] = in[g];
  }
  FLUXMI_REQUIRE(aligned16(out), FLUXMI_ERR_INVALID_ARG,
                 "topk_gather_reduce: output is not 16-byte aligned");
  if (ntokens == 0 || n == 0) return FLUXMI_OK;

  const int32_t nvec = n / 8;
  FLUXMI_REQUIRE(static_cast<int64_t>(ntokens) * topk <= INT32_MAX, FLUXMI_ERR_UNSUPPORTED,
                 "topk_gather_reduce: ntokens*topk exceeds 2^31-1");
  const int32_t nrows = ntokens * topk;  // rows of every input matrix
  // One workgroup per token row; rows wider than 2 vectors per lane are split over blockIdx.y so
  // that small token counts still fill the chip.
  const int threads = nvec >= 512 ? 512 : 256;
  int ysplit = 1;
  if (ntokens < 2048) {
    ysplit = (nvec + threads - 1) / threads;
    if (ysplit > 16) ysplit = 16;
  }
  const size_t in_bytes = static_cast<size_t>(ntokens) * topk * n * (in_fp32 ? 4 : 2) * ngroups;
  const int nt = in_bytes > kPlainLoadMaxBytes ? 1 : 0;
  const dim3 grid(static_cast<unsigned>(ntokens), static_cast<unsigned>(ysplit));
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool weighted = row_weight != nullptr;
  uint16_t *o = static_cast<uint16_t *>(out);
  switch (ngroups) {
    case 1: dispatch_topk<1>(weighted, in_fp32 != 0, grid, threads, nt, s, gp, routing_idx, row_weight, scale, topk, nvec, nrows, o, half_f16); break;
    case 2: dispatch_topk<2>(weighted, in_fp32 != 0, grid, threads, nt, s, gp, routing_idx, row_weight, scale, topk, nvec, nrows, o, half_f16); break;
    case 3: dispatch_topk<3>(weighted, in_fp32 != 0, grid, threads, nt, s, gp, routing_idx, row_weight, scale, topk, nvec, nrows, o, half_f16); break;
    default: dispatch_topk<4>(weighted, in_fp32 != 0, grid, threads, nt, s, gp, routing_idx, row_weight, scale, topk, nvec, nrows, o, half_f16); break;
  }
  FLUXMI_HIP_CHECK(hipGetLastError());
  return FLUXMI_OK;
}
