// bf16 -> fp8-e4m3 absmax quantisation with one scale per row, per (row, 128-column block) or per
// 128 x 128 block (with an optional transposed copy of the bytes).
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

// ---- one scale per 128 x 128 block, optional transposed copy -----------------------------------
// One workgroup per block.  Lane (rg, cg) = (tid / 16, tid % 16) holds the 8 x 8 patch at rows
// rg*8.., columns cg*8.. of the block in registers between the amax pass and the cast pass: a load
// instruction of a wave covers 4 x 256 contiguous bytes.  The transposed copy goes through LDS: each
// lane transposes its 8 x 8 patch of bytes in registers, writes eight 8-byte pieces (piece p of
// transposed row c at slot p ^ (c / 8): spreads the 16 lanes that share p over the banks), and the
// workgroup reads the 128 transposed rows back 16 bytes per lane, 8 lanes per row.
// VEC: cols % 8 == 0 and aligned pointers (16-byte loads, 8-byte stores); else element accesses.
// VEC_T: rows % 16 == 0 and q_t aligned (16-byte stores of the transposed rows); else byte stores.
template <bool VEC, bool TRANSPOSE, bool VEC_T>
__global__ __launch_bounds__(256) void quant_square_kernel(const uint16_t *__restrict__ x, int64_t rows,
                                                           int64_t cols, int32_t nbx, int32_t nby,
                                                           float eps, uint8_t *__restrict__ q,
                                                           float *__restrict__ scale_inv,
                                                           uint8_t *__restrict__ q_t,
                                                           float *__restrict__ scale_inv_t) {
  __shared__ uint32_t s_amax[4];
  __shared__ __attribute__((aligned(16))) uint8_t s_t[TRANSPOSE ? 128 * 128 : 16];
  const int bx = blockIdx.x % nbx;
  const int by = (blockIdx.x / nbx) % nby;
  const int64_t b = blockIdx.x / (nbx * nby);
  const int cg = threadIdx.x & 15, rg = threadIdx.x >> 4;
  const int64_t r0 = static_cast<int64_t>(by) * 128 + rg * 8;
  const int64_t c0 = static_cast<int64_t>(bx) * 128 + cg * 8;
  const uint16_t *xb = x + b * rows * cols;
  uint8_t *qb = q + b * rows * cols;

  u32x4 v[8];
  uint32_t m = 0u;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    v[i] = u32x4{0u, 0u, 0u, 0u};  // what lies outside the matrix counts as zero
    const int64_t r = r0 + i;
    if (r < rows) {
      if constexpr (VEC) {
        if (c0 < cols) v[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(xb + r * cols + c0));
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (c0 + e < cols) v[i][e >> 1] |= static_cast<uint32_t>(xb[r * cols + c0 + e]) << ((e & 1) * 16);
      }
    }
    m = max(m, amax8(v[i]));
  }
  m = wave_max_u32(m);
  if ((threadIdx.x & 63) == 0) s_amax[threadIdx.x >> 6] = m;
  __syncthreads();
  m = max(max(s_amax[0], s_amax[1]), max(s_amax[2], s_amax[3]));
  const float scale = compute_scale(__uint_as_float(m), eps);
  if (threadIdx.x == 0) {
    const float inv = 1.0f / scale;  // fp32 division (src/quantization/quantization.cu:1117)
    scale_inv[(b * nby + by) * nbx + bx] = inv;
    if constexpr (TRANSPOSE) scale_inv_t[(b * nbx + bx) * nby + by] = inv;
  }

  u32x2 o[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    o[i] = cast8(v[i], scale);
    const int64_t r = r0 + i;
    if (r < rows) {
      if constexpr (VEC) {
        if (c0 < cols) __builtin_nontemporal_store(o[i], reinterpret_cast<u32x2 *>(qb + r * cols + c0));
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (c0 + e < cols) qb[r * cols + c0 + e] = static_cast<uint8_t>(o[i][e >> 2] >> ((e & 3) * 8));
      }
    }
  }

  if constexpr (TRANSPOSE) {
    uint8_t *qtb = q_t + b * rows * cols;
#pragma unroll
    for (int j = 0; j < 8; ++j) {  // column j of the patch: byte j of each of the eight rows
      u32x2 t;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        uint32_t w = 0u;
#pragma unroll
        for (int i = 0; i < 4; ++i) w |= ((o[4 * h + i][j >> 2] >> ((j & 3) * 8)) & 0xffu) << (8 * i);
        t[h] = w;
      }
      *reinterpret_cast<u32x2 *>(s_t + (cg * 8 + j) * 128 + ((rg ^ cg) * 8)) = t;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int vid = threadIdx.x + 256 * k;
      const int trow = vid >> 3, pp = vid & 7;  // transposed row (a column of x), 16-byte unit in it
      const int tcg = trow >> 3;
      // Pieces 2pp and 2pp+1 sit in slots (2pp ^ tcg) and (2pp ^ tcg) ^ 1: one aligned 16-byte unit,
      // its halves swapped when tcg is odd.
      u32x4 d = *reinterpret_cast<const u32x4 *>(s_t + trow * 128 + (((2 * pp) ^ tcg) & ~1) * 8);
      if (tcg & 1) d = u32x4{d[2], d[3], d[0], d[1]};
      const int64_t c = static_cast<int64_t>(bx) * 128 + trow;
      const int64_t r = static_cast<int64_t>(by) * 128 + pp * 16;
      if (c < cols && r < rows) {
        if constexpr (VEC_T) {
          __builtin_nontemporal_store(d, reinterpret_cast<u32x4 *>(qtb + c * rows + r));
        } else {
#pragma unroll
          for (int e = 0; e < 16; ++e)
            if (r + e < rows) qtb[c * rows + r + e] = static_cast<uint8_t>(d[e >> 2] >> ((e & 3) * 8));
        }
      }
    }
  }
}

// ---- one scale per (row, 128-column block), optional transposed copy with its own scales --------
// Same workgroup shape as the 128 x 128 kernel: lane (rg, cg) holds an 8 x 8 patch.  Row direction: the
// 16 lanes of a row segment reduce its amax with four xor shuffles.  Column direction (the transposed
// output: one scale per column and 128-row block): 8 in-lane maxima per column, two xor shuffles across
// the four row groups of a wave, LDS across the four waves.  Both outputs come from one read of x.
// Scales are stored as [ceil(rows/128)][ceil(cols/128)][128] (row inside its block fastest), the
// transposed ones as [ceil(cols/128)][ceil(rows/128)][128].  scale_inv is the fp32 quotient 1.0f / scale:
// equal to the reference's float(1.0 / double(scale)), since a quotient rounded to 53 bits and then to 24
// (or fewer, for a denormal result) is the correctly rounded quotient.
__device__ __forceinline__ float bf16_elem(const u32x4 v, int e) {
  return __uint_as_float((e & 1) ? (v[e >> 1] & 0xffff0000u) : (v[e >> 1] << 16));
}

// With the transposed output the kernel is a chain of dependent phases; four waves per SIMD (128 registers,
// a few spilled) hide them better than the two the unconstrained allocation leaves.
template <bool VEC, bool TRANSPOSE, bool VEC_T>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(TRANSPOSE ? 4 : 1, TRANSPOSE ? 4 : 8)))
void quant_block128_tile_kernel(const uint16_t *__restrict__ x, int64_t rows,
                                                                  int64_t cols, int32_t nbx, int32_t nby,
                                                                  float eps, uint8_t *__restrict__ q,
                                                                  float *__restrict__ scale_inv,
                                                                  uint8_t *__restrict__ q_t,
                                                                  float *__restrict__ scale_inv_t) {
  __shared__ __attribute__((aligned(16))) uint32_t s_col[TRANSPOSE ? 4 * 128 : 4];
  __shared__ __attribute__((aligned(16))) uint8_t s_t[TRANSPOSE ? 128 * 128 : 16];
  const int bx = blockIdx.x % nbx;
  const int by = blockIdx.x / nbx;
  const int cg = threadIdx.x & 15, rg = threadIdx.x >> 4;
  const int64_t r0 = static_cast<int64_t>(by) * 128 + rg * 8;
  const int64_t c0 = static_cast<int64_t>(bx) * 128 + cg * 8;

  u32x4 v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    v[i] = u32x4{0u, 0u, 0u, 0u};  // what lies outside the matrix counts as zero
    const int64_t r = r0 + i;
    if (r < rows) {
      if constexpr (VEC) {
        if (c0 < cols) v[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(x + r * cols + c0));
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (c0 + e < cols) v[i][e >> 1] |= static_cast<uint32_t>(x[r * cols + c0 + e]) << ((e & 1) * 16);
      }
    }
  }

  if constexpr (TRANSPOSE) {  // column maxima first: their way through LDS overlaps the row-direction work
    uint32_t cm[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      uint32_t m = 0u;
#pragma unroll
      for (int i = 0; i < 8; ++i)
        m = max(m, abs_bits_skip_nan((j & 1) ? (v[i][j >> 1] & 0xffff0000u) : (v[i][j >> 1] << 16)));
      m = max(m, static_cast<uint32_t>(__shfl_xor(static_cast<int>(m), 16, 64)));
      m = max(m, static_cast<uint32_t>(__shfl_xor(static_cast<int>(m), 32, 64)));
      cm[j] = m;
    }
    if ((threadIdx.x & 48) == 0) {
      uint32_t *dst = s_col + (threadIdx.x >> 6) * 128 + cg * 8;
      *reinterpret_cast<u32x4 *>(dst) = u32x4{cm[0], cm[1], cm[2], cm[3]};
      *reinterpret_cast<u32x4 *>(dst + 4) = u32x4{cm[4], cm[5], cm[6], cm[7]};
    }
  }

#pragma unroll
  for (int i = 0; i < 8; ++i) {
    uint32_t m = amax8(v[i]);
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) m = max(m, static_cast<uint32_t>(__shfl_xor(static_cast<int>(m), off, 64)));
    const float scale = compute_scale(__uint_as_float(m), eps);
    const int64_t r = r0 + i;
    if (r < rows) {
      if (cg == 0)
        scale_inv[static_cast<int64_t>(by) * (static_cast<int64_t>(nbx) * 128) + static_cast<int64_t>(bx) * 128 +
                  (r & 127)] = 1.0f / scale;
      const u32x2 o = cast8(v[i], scale);
      if constexpr (VEC) {
        if (c0 < cols) __builtin_nontemporal_store(o, reinterpret_cast<u32x2 *>(q + r * cols + c0));
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (c0 + e < cols) q[r * cols + c0 + e] = static_cast<uint8_t>(o[e >> 2] >> ((e & 3) * 8));
      }
    }
  }

  if constexpr (TRANSPOSE) {
    __syncthreads();
    u32x4 ca = u32x4{0u, 0u, 0u, 0u}, cb = ca;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const u32x4 a = *reinterpret_cast<const u32x4 *>(s_col + w * 128 + cg * 8);
      const u32x4 b = *reinterpret_cast<const u32x4 *>(s_col + w * 128 + cg * 8 + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        ca[e] = max(ca[e], a[e]);
        cb[e] = max(cb[e], b[e]);
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float scale = compute_scale(__uint_as_float(j < 4 ? ca[j & 3] : cb[j & 3]), eps);
      const int64_t c = c0 + j;
      if (rg == 0 && c < cols)
        scale_inv_t[static_cast<int64_t>(bx) * (static_cast<int64_t>(nby) * 128) + static_cast<int64_t>(by) * 128 +
                    (c & 127)] = 1.0f / scale;
      u32x2 t;
#pragma unroll
      for (int h = 0; h < 2; ++h)
        t[h] = pack2_e4m3(bf16_elem(v[4 * h], j) * scale, bf16_elem(v[4 * h + 1], j) * scale) |
               (pack2_e4m3(bf16_elem(v[4 * h + 2], j) * scale, bf16_elem(v[4 * h + 3], j) * scale) << 16);
      *reinterpret_cast<u32x2 *>(s_t + (cg * 8 + j) * 128 + ((rg ^ cg) * 8)) = t;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int vid = threadIdx.x + 256 * k;
      const int trow = vid >> 3, pp = vid & 7;
      const int tcg = trow >> 3;
      u32x4 d = *reinterpret_cast<const u32x4 *>(s_t + trow * 128 + (((2 * pp) ^ tcg) & ~1) * 8);
      if (tcg & 1) d = u32x4{d[2], d[3], d[0], d[1]};
      const int64_t c = static_cast<int64_t>(bx) * 128 + trow;
      const int64_t r = static_cast<int64_t>(by) * 128 + pp * 16;
      if (c < cols && r < rows) {
        if constexpr (VEC_T) {
          __builtin_nontemporal_store(d, reinterpret_cast<u32x4 *>(q_t + c * rows + r));
        } else {
#pragma unroll
          for (int e = 0; e < 16; ++e)
            if (r + e < rows) q_t[c * rows + r + e] = static_cast<uint8_t>(d[e >> 2] >> ((e & 3) * 8));
        }
      }
    }
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

  if (block_cols == 128 && permute_scale) {
    // The reference's layout: the tile kernel (faster than walking rows: eight loads in flight per lane).
    return fluxmi_quant_e4m3_block128(x_bf16, rows, cols, eps, q_out, scale_inv_out, nullptr, nullptr, stream);
  }
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

extern "C" int fluxmi_quant_e4m3_square(const void *x_bf16, int64_t batch, int64_t rows, int64_t cols,
                                        float eps, void *q_out, float *scale_inv_out, void *q_t_out,
                                        float *scale_inv_t_out, void *stream) {
  using namespace fluxmi;
  FLUXMI_REQUIRE(x_bf16 != nullptr && q_out != nullptr && scale_inv_out != nullptr,
                 FLUXMI_ERR_INVALID_ARG, "quant_e4m3_square: null pointer argument");
  FLUXMI_REQUIRE((q_t_out == nullptr) == (scale_inv_t_out == nullptr), FLUXMI_ERR_INVALID_ARG,
                 "quant_e4m3_square: q_t_out and scale_inv_t_out go together");
  FLUXMI_REQUIRE(batch >= 0 && rows >= 0 && cols >= 0, FLUXMI_ERR_INVALID_ARG,
                 "quant_e4m3_square: negative size (batch=%lld, rows=%lld, cols=%lld)",
                 static_cast<long long>(batch), static_cast<long long>(rows), static_cast<long long>(cols));
  FLUXMI_REQUIRE((reinterpret_cast<uintptr_t>(x_bf16) & 1u) == 0, FLUXMI_ERR_INVALID_ARG,
                 "quant_e4m3_square: x must be 2-byte aligned");
  if (batch == 0 || rows == 0 || cols == 0) return FLUXMI_OK;
  const int64_t nbx = (cols + 127) / 128, nby = (rows + 127) / 128;
  FLUXMI_REQUIRE(nbx <= INT32_MAX && nby <= INT32_MAX && batch <= INT32_MAX &&
                     nbx * nby <= INT32_MAX / batch,
                 FLUXMI_ERR_UNSUPPORTED, "quant_e4m3_square: more than 2^31 blocks");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uint16_t *x = static_cast<const uint16_t *>(x_bf16);
  uint8_t *q = static_cast<uint8_t *>(q_out);
  uint8_t *qt = static_cast<uint8_t *>(q_t_out);
  const dim3 grid(static_cast<unsigned>(batch * nbx * nby)), block(256);
  const bool vec = cols % 8 == 0 && aligned16(x_bf16) && (reinterpret_cast<uintptr_t>(q_out) & 7u) == 0;
  const bool vec_t = rows % 16 == 0 && aligned16(q_t_out);
#define FLUXMI_SQ(V, T, VT)                                                                            \
  hipLaunchKernelGGL((quant_square_kernel<V, T, VT>), grid, block, 0, s, x, rows, cols,                \
                     static_cast<int32_t>(nbx), static_cast<int32_t>(nby), eps, q, scale_inv_out, qt,  \
                     scale_inv_t_out)
  if (qt == nullptr) {
    if (vec) FLUXMI_SQ(true, false, false);
    else FLUXMI_SQ(false, false, false);
  } else if (vec) {
    if (vec_t) FLUXMI_SQ(true, true, true);
    else FLUXMI_SQ(true, true, false);
  } else {
    if (vec_t) FLUXMI_SQ(false, true, true);
    else FLUXMI_SQ(false, true, false);
  }
#undef FLUXMI_SQ
  FLUXMI_HIP_CHECK(hipGetLastError());
  return FLUXMI_OK;
}

extern "C" int fluxmi_quant_e4m3_block128(const void *x_bf16, int64_t rows, int64_t cols, float eps,
                                          void *q_out, float *scale_inv_out, void *q_t_out,
                                          float *scale_inv_t_out, void *stream) {
  using namespace fluxmi;
  FLUXMI_REQUIRE(x_bf16 != nullptr && q_out != nullptr && scale_inv_out != nullptr,
                 FLUXMI_ERR_INVALID_ARG, "quant_e4m3_block128: null pointer argument");
  FLUXMI_REQUIRE((q_t_out == nullptr) == (scale_inv_t_out == nullptr), FLUXMI_ERR_INVALID_ARG,
                 "quant_e4m3_block128: q_t_out and scale_inv_t_out go together");
  FLUXMI_REQUIRE(rows >= 0 && cols >= 0, FLUXMI_ERR_INVALID_ARG,
                 "quant_e4m3_block128: negative size (rows=%lld, cols=%lld)", static_cast<long long>(rows),
                 static_cast<long long>(cols));
  FLUXMI_REQUIRE((reinterpret_cast<uintptr_t>(x_bf16) & 1u) == 0, FLUXMI_ERR_INVALID_ARG,
                 "quant_e4m3_block128: x must be 2-byte aligned");
  if (rows == 0 || cols == 0) return FLUXMI_OK;
  const int64_t nbx = (cols + 127) / 128, nby = (rows + 127) / 128;
  FLUXMI_REQUIRE(nbx <= INT32_MAX && nby <= INT32_MAX && nbx * nby <= INT32_MAX, FLUXMI_ERR_UNSUPPORTED,
                 "quant_e4m3_block128: more than 2^31 blocks");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uint16_t *x = static_cast<const uint16_t *>(x_bf16);
  uint8_t *q = static_cast<uint8_t *>(q_out);
  uint8_t *qt = static_cast<uint8_t *>(q_t_out);
  const dim3 grid(static_cast<unsigned>(nbx * nby)), block(256);
  const bool vec = cols % 8 == 0 && aligned16(x_bf16) && (reinterpret_cast<uintptr_t>(q_out) & 7u) == 0;
  const bool vec_t = rows % 16 == 0 && aligned16(q_t_out);
#define FLUXMI_B128(V, T, VT)                                                                          \
  hipLaunchKernelGGL((quant_block128_tile_kernel<V, T, VT>), grid, block, 0, s, x, rows, cols,         \
                     static_cast<int32_t>(nbx), static_cast<int32_t>(nby), eps, q, scale_inv_out, qt,  \
                     scale_inv_t_out)
  if (qt == nullptr) {
    if (vec) FLUXMI_B128(true, false, false);
    else FLUXMI_B128(false, false, false);
  } else if (vec) {
    if (vec_t) FLUXMI_B128(true, true, true);
    else FLUXMI_B128(true, true, false);
  } else {
    if (vec_t) FLUXMI_B128(false, true, true);
    else FLUXMI_B128(false, true, false);
  }
#undef FLUXMI_B128
  FLUXMI_HIP_CHECK(hipGetLastError());
  return FLUXMI_OK;
}
