// bf16 -> fp8-e4m3 absmax quantisation with one scale per row or per (row, 128-column block).
//
// HBM-streaming kernel: one read of x (2 B/elt), one write of q (1 B/elt).  A row (or row block) is
// held in registers between the amax pass and the cast pass, so x is fetched exactly once.
#include "common.hpp"

namespace fluxmi {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr float kE4M3Max = 448.f;

// scale = 448 / max(amax, eps) with the special cases of the reference's ComputeScale
// (src/quantization/quantization.cu:306-367, bf16 input type, no power-of-two rounding).
__device__ __forceinline__ float compute_scale(float amax, float eps) {
  const float a = fmaxf(amax, eps);
  if (a == 0.f) return 1.f;
  const float s = kE4M3Max / a;  // IEEE fp32 division
  if (__builtin_isinf(s)) return 0x1.FEp127f;
  return s;  // includes s == 0 when amax is +inf
}

#ifdef FLUXMI_SOFT_FP8
// Bit-level fp32 -> e4m3 (OCP "fn"): round to nearest even, saturate to +-448, NaN -> 0x7f.
__device__ __forceinline__ uint32_t f32_to_e4m3(float f) {
  const uint32_t u = __float_as_uint(f);
  const uint32_t sign = (u >> 24) & 0x80u;
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return sign | 0x7fu;
  if (a >= 0x43e00000u) return sign | 0x7eu;  // |f| >= 448
  if (a < 0x3c800000u) {                      // |f| < 2^-6: subnormal grid of 2^-9
    const float q = __builtin_rintf(__uint_as_float(a) * 512.f);
    return sign | static_cast<uint32_t>(q);
  }
  a += 0x7ffffu + ((a >> 20) & 1u);
  return sign | ((a >> 20) - (120u << 3));
}
__device__ __forceinline__ uint32_t pack2_e4m3(float lo, float hi) {
  return f32_to_e4m3(lo) | (f32_to_e4m3(hi) << 8);
}
#else
// Hardware conversion (v_cvt_pk_fp8_f32, OCP e4m3 on gfx950, round to nearest even).  The operands are
// clamped first so that the result saturates whatever the conversion's own overflow rule is; NaN
// passes through the clamp untouched.
__device__ __forceinline__ float clamp448(float f) {
  const float c = fminf(fmaxf(f, -kE4M3Max), kE4M3Max);
  return f != f ? f : c;
}
__device__ __forceinline__ uint32_t pack2_e4m3(float lo, float hi) {
  return static_cast<uint32_t>(__builtin_amdgcn_cvt_pk_fp8_f32(clamp448(lo), clamp448(hi), 0, false)) &
         0xffffu;
}
#endif

// Largest |x| of 8 bf16 values as fp32 bits.  Done on the integer patterns (for non-negative floats the
// unsigned order is the numeric order) so that every NaN, signalling ones included, is skipped exactly
// as CUDA's fmaxf skips it; +-inf takes part.
__device__ __forceinline__ uint32_t abs_bits_skip_nan(uint32_t f32_bits) {
  const uint32_t a = f32_bits & 0x7fffffffu;
  return a > 0x7f800000u ? 0u : a;
}
__device__ __forceinline__ uint32_t amax8(const u32x4 v) {
  uint32_t m = 0u;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    m = max(m, abs_bits_skip_nan(v[i] << 16));
    m = max(m, abs_bits_skip_nan(v[i] & 0xffff0000u));
  }
  return m;
}
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = max(v, static_cast<uint32_t>(__shfl_xor(static_cast<int>(v), off, 64)));
  return v;
}

__device__ __forceinline__ u32x2 cast8(const u32x4 v, const float scale) {
  u32x2 o;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const float f0 = __uint_as_float(v[2 * h] << 16) * scale;
    const float f1 = __uint_as_float(v[2 * h] & 0xffff0000u) * scale;
    const float f2 = __uint_as_float(v[2 * h + 1] << 16) * scale;
    const float f3 = __uint_as_float(v[2 * h + 1] & 0xffff0000u) * scale;
    o[h] = pack2_e4m3(f0, f1) | (pack2_e4m3(f2, f3) << 16);
  }
  return o;
}

// ---- one scale per row -------------------------------------------------------------------------
// THREADS_PER_ROW lanes (64, 128 or 256) cooperate on one row; a 256-thread workgroup therefore
// handles 256/THREADS_PER_ROW rows.  Each lane keeps up to VPT 16-byte vectors in registers.
template <int THREADS_PER_ROW, int VPT>
__global__ __launch_bounds__(256) void quant_row_kernel(const uint16_t *__restrict__ x, int64_t rows,
                                                        int32_t nvec, float eps,
                                                        uint8_t *__restrict__ q,
                                                        float *__restrict__ scale_inv) {
  constexpr int kRowsPerBlock = 256 / THREADS_PER_ROW;
  constexpr int kWavesPerRow = THREADS_PER_ROW / 64;
  __shared__ uint32_t s_amax[4];
  const int sub = threadIdx.x / THREADS_PER_ROW;
  const int tid = threadIdx.x % THREADS_PER_ROW;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock + sub;
  const bool row_ok = row < rows;
  const u32x4 *src = reinterpret_cast<const u32x4 *>(x) + (row_ok ? row : 0) * nvec;

  u32x4 v[VPT];
  uint32_t m = 0u;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int c = tid + i * THREADS_PER_ROW;
    v[i] = u32x4{0u, 0u, 0u, 0u};
    if (row_ok && c < nvec) v[i] = __builtin_nontemporal_load(src + c);
    m = max(m, amax8(v[i]));
  }
  m = wave_max_u32(m);
  if constexpr (kWavesPerRow > 1) {
    const int wave = threadIdx.x / 64;
    if ((threadIdx.x & 63) == 0) s_amax[wave] = m;
    __syncthreads();
    const int w0 = sub * kWavesPerRow;
#pragma unroll
    for (int w = 0; w < kWavesPerRow; ++w) m = max(m, s_amax[w0 + w]);
  }
  const float scale = compute_scale(__uint_as_float(m), eps);
  if (!row_ok) return;
  if (tid == 0) scale_inv[row] = static_cast<float>(1.0 / static_cast<double>(scale));
  u32x2 *dst = reinterpret_cast<u32x2 *>(q) + row * nvec;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int c = tid + i * THREADS_PER_ROW;
    if (c < nvec) __builtin_nontemporal_store(cast8(v[i], scale), dst + c);
  }
}

// Rows too long for the register-resident kernel: two passes over the row (the second hits L2).
__global__ __launch_bounds__(256) void quant_row_long_kernel(const uint16_t *__restrict__ x,
                                                             int64_t rows, int32_t nvec, float eps,
                                                             uint8_t *__restrict__ q,
                                                             float *__restrict__ scale_inv) {
  __shared__ uint32_t s_amax[4];
  const int64_t row = blockIdx.x;
  const u32x4 *src = reinterpret_cast<const u32x4 *>(x) + row * nvec;
  uint32_t m = 0u;
  for (int c = threadIdx.x; c < nvec; c += 256) m = max(m, amax8(src[c]));
  m = wave_max_u32(m);
  if ((threadIdx.x & 63) == 0) s_amax[threadIdx.x / 64] = m;
  __syncthreads();
  m = max(max(s_amax[0], s_amax[1]), max(s_amax[2], s_amax[3]));
  const float scale = compute_scale(__uint_as_float(m), eps);
  if (threadIdx.x == 0) scale_inv[row] = static_cast<float>(1.0 / static_cast<double>(scale));
  u32x2 *dst = reinterpret_cast<u32x2 *>(q) + row * nvec;
  for (int c = threadIdx.x; c < nvec; c += 256) dst[c] = cast8(src[c], scale);
}

// ---- one scale per (row, 128-column block) -----------------------------------------------------
// 16 consecutive lanes own one block (16 vectors of 8 elements); the amax reduction is four xor
// shuffles inside that lane group.
template <int THREADS_PER_ROW>
__global__ __launch_bounds__(256) void quant_block128_kernel(const uint16_t *__restrict__ x,
                                                             int64_t rows, int32_t nvec,
                                                             int32_t nblocks, float eps,
                                                             uint8_t *__restrict__ q,
                                                             float *__restrict__ scale_inv,
                                                             int32_t permute) {
  // THREADS_PER_ROW lanes walk one row in steps of THREADS_PER_ROW vectors; blocks start at multiples
  // of 16 vectors, so the 16 lanes of a block always step together.
  constexpr int kRowsPerBlock = 256 / THREADS_PER_ROW;
  const int tid = threadIdx.x % THREADS_PER_ROW;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock + threadIdx.x / THREADS_PER_ROW;
  if (row >= rows) return;
  const u32x4 *src = reinterpret_cast<const u32x4 *>(x) + row * nvec;
  u32x2 *dst = reinterpret_cast<u32x2 *>(q) + row * nvec;
  for (int c = tid; c < nblocks * 16; c += THREADS_PER_ROW) {
    const bool ok = c < nvec;  // a partial last block: missing vectors count as zeros
    u32x4 v = u32x4{0u, 0u, 0u, 0u};
    if (ok) v = __builtin_nontemporal_load(src + c);
    uint32_t m = amax8(v);
#pragma unroll
    for (int off = 8; off > 0; off >>= 1)
      m = max(m, static_cast<uint32_t>(__shfl_xor(static_cast<int>(m), off, 64)));
    const float scale = compute_scale(__uint_as_float(m), eps);
    if ((c & 15) == 0) {
      const int blk = c >> 4;
      const float inv = static_cast<float>(1.0 / static_cast<double>(scale));
      if (permute)
        scale_inv[(row >> 7) * (static_cast<int64_t>(nblocks) * 128) + static_cast<int64_t>(blk) * 128 +
                  (row & 127)] = inv;
      else
        scale_inv[row * nblocks + blk] = inv;
    }
    if (ok) __builtin_nontemporal_store(cast8(v, scale), dst + c);
  }
}

template <int TPR>
void launch_block128(hipStream_t s, const uint16_t *x, int64_t rows, int32_t nvec, int32_t nblocks, float eps,
                     uint8_t *q, float *si, int32_t permute) {
  constexpr int kRowsPerBlock = 256 / TPR;
  const unsigned grid = static_cast<unsigned>((rows + kRowsPerBlock - 1) / kRowsPerBlock);
  hipLaunchKernelGGL((quant_block128_kernel<TPR>), dim3(grid), dim3(256), 0, s, x, rows, nvec, nblocks, eps, q, si,
                     permute);
}

template <int TPR, int VPT>
void launch_row(hipStream_t s, const uint16_t *x, int64_t rows, int32_t nvec, float eps, uint8_t *q,
                float *si) {
  constexpr int kRowsPerBlock = 256 / TPR;
  const unsigned grid = static_cast<unsigned>((rows + kRowsPerBlock - 1) / kRowsPerBlock);
  hipLaunchKernelGGL((quant_row_kernel<TPR, VPT>), dim3(grid), dim3(256), 0, s, x, rows, nvec, eps, q,
                     si);
}

}  // namespace
}  // namespace fluxmi

extern "C" int fluxmi_quant_e4m3_rowwise(const void *x_bf16, int64_t rows, int64_t cols,
                                         int32_t block_cols, float eps, void *q_out,
                                         float *scale_inv_out, int32_t permute_scale, void *stream) {
  using namespace fluxmi;
  FLUXMI_REQUIRE(x_bf16 != nullptr && q_out != nullptr && scale_inv_out != nullptr,
                 FLUXMI_ERR_INVALID_ARG, "quant_e4m3_rowwise: null pointer argument");
  FLUXMI_REQUIRE(rows >= 0 && cols >= 0, FLUXMI_ERR_INVALID_ARG,
                 "quant_e4m3_rowwise: negative size (rows=%lld, cols=%lld)",
                 static_cast<long long>(rows), static_cast<long long>(cols));
  FLUXMI_REQUIRE(block_cols == 0 || block_cols == 128, FLUXMI_ERR_UNSUPPORTED,
                 "quant_e4m3_rowwise: block_cols=%d (0 = whole row, or 128)", block_cols);
  FLUXMI_REQUIRE(cols % 8 == 0, FLUXMI_ERR_UNSUPPORTED,
                 "quant_e4m3_rowwise: cols=%lld is not a multiple of 8", static_cast<long long>(cols));
  FLUXMI_REQUIRE(cols / 8 <= INT32_MAX && rows <= (int64_t{1} << 40), FLUXMI_ERR_UNSUPPORTED,
                 "quant_e4m3_rowwise: matrix too large");
  FLUXMI_REQUIRE(aligned16(x_bf16) && (reinterpret_cast<uintptr_t>(q_out) & 7u) == 0,
                 FLUXMI_ERR_INVALID_ARG, "quant_e4m3_rowwise: x must be 16-byte and q 8-byte aligned");
  if (rows == 0 || cols == 0) return FLUXMI_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uint16_t *x = static_cast<const uint16_t *>(x_bf16);
  uint8_t *q = static_cast<uint8_t *>(q_out);
  const int32_t nvec = static_cast<int32_t>(cols / 8);

  if (block_cols == 128) {
    const int32_t nblocks = static_cast<int32_t>((cols + 127) / 128);
    FLUXMI_REQUIRE(rows <= INT32_MAX, FLUXMI_ERR_UNSUPPORTED, "quant_e4m3_rowwise: too many rows");
    const int32_t lanes = nblocks * 16;
    if (lanes <= 64) launch_block128<64>(s, x, rows, nvec, nblocks, eps, q, scale_inv_out, permute_scale);
    else if (lanes <= 128) launch_block128<128>(s, x, rows, nvec, nblocks, eps, q, scale_inv_out, permute_scale);
    else launch_block128<256>(s, x, rows, nvec, nblocks, eps, q, scale_inv_out, permute_scale);
  } else {
    FLUXMI_REQUIRE(rows <= INT32_MAX, FLUXMI_ERR_UNSUPPORTED, "quant_e4m3_rowwise: too many rows");
    if (nvec <= 64) launch_row<64, 1>(s, x, rows, nvec, eps, q, scale_inv_out);
    else if (nvec <= 128) launch_row<64, 2>(s, x, rows, nvec, eps, q, scale_inv_out);
    else if (nvec <= 256) launch_row<64, 4>(s, x, rows, nvec, eps, q, scale_inv_out);
    else if (nvec <= 512) launch_row<128, 4>(s, x, rows, nvec, eps, q, scale_inv_out);
    else if (nvec <= 1024) launch_row<256, 4>(s, x, rows, nvec, eps, q, scale_inv_out);
    else if (nvec <= 2048) launch_row<256, 8>(s, x, rows, nvec, eps, q, scale_inv_out);
    else
      hipLaunchKernelGGL(quant_row_long_kernel, dim3(static_cast<unsigned>(rows)), dim3(256), 0, s, x,
                         rows, nvec, eps, q, scale_inv_out);
  }
  FLUXMI_HIP_CHECK(hipGetLastError());
  return FLUXMI_OK;
}
