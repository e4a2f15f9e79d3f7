/*
 * CPU restatement (plain C) of the arithmetic of bytedance/flux's bf16 -> fp8-e4m3 block-scaled cast.
 * TEST INFRASTRUCTURE ONLY: built into oracle/_build/libquant_ref.so and loaded by tests / bench.
 *
 * Follows src/quantization/quantization.cu:
 *   ComputeScale            :306-367  (scale = fp8_max / max(amax, eps); 0 -> 1; inf -> bf16 max; no pow2)
 *   F8LimitsTrait e4m3      :232-235  (448)
 *   bf16 "max" on overflow  :262-266  (0x1.FEp127)
 *   scale_inv = 1.0 / scale :612-621  (double division, stored as float; permuted [M/128][K/128][128])
 *   q = OType(float(x)*scale):674-676 (CUDA __nv_fp8_e4m3 constructor: round-nearest-even, saturate-finite)
 *   padding counts as 0     :519-525
 *   128 x 128 blocks        :971-1183 (ragged), :1185-1380 (full); scale_inv = 1.0f / scale :1117, :1290
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static float bits_to_float(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static uint32_t float_to_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}

/* CUDA's fmaxf: a NaN operand is ignored (the other operand is returned). Written out so that no
 * compiler lowering of fmaxf to a NaN-propagating max instruction can change it. */
static float max_ignore_nan(float a, float b) {
  if (b != b) return a;
  if (a != a) return b;
  return a > b ? a : b;
}

float fluxref_compute_scale(float amax, float eps) {
  float amax_mod = max_ignore_nan(amax, eps);
  if (amax_mod == 0.f) return 1.f;
  float scale = 448.0f / amax_mod;
  if (isinf(scale)) return 0x1.FEp127f;
  return scale; /* scale == 0 (amax = inf) is returned as is */
}

/* OCP e4m3 ("fn": no inf, 0x7f/0xff = NaN): round to nearest even, saturate to +-448. */
uint8_t fluxref_f32_to_e4m3(float f) {
  uint32_t u = float_to_bits(f);
  uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint8_t)(sign | 0x7f);
  float af = bits_to_float(a);
  if (af >= 448.0f) return (uint8_t)(sign | 0x7e);
  if (af < 0x1p-6f) { /* subnormal grid: multiples of 2^-9, ties to even */
    float q = nearbyintf(af * 512.0f);
    return (uint8_t)(sign | (uint8_t)q);
  }
  int ex;
  float m = frexpf(af, &ex);            /* af = m * 2^ex, m in [0.5, 1) */
  float q = nearbyintf(m * 16.0f);      /* 4 significant bits (1 + 3 mantissa), ties to even */
  if (q == 16.0f) {
    q = 8.0f;
    ex += 1;
  }
  int e = ex - 1 + 7;                   /* biased exponent, value = (q/8) * 2^(ex-1) */
  return (uint8_t)(sign | (uint8_t)(e << 3) | ((uint8_t)q & 7u));
}

float fluxref_e4m3_to_f32(uint8_t b) {
  int sign = b & 0x80;
  int e = (b >> 3) & 0xf;
  int m = b & 7;
  float v;
  if (e == 0xf && m == 7) return NAN;
  if (e == 0) v = ldexpf((float)m, -9);
  else v = ldexpf((float)(8 + m), e - 7 - 3);
  return sign ? -v : v;
}

static float bf16_to_f32(uint16_t h) { return bits_to_float((uint32_t)h << 16); }

/* block_cols == 0: one scale per row, scale_inv[rows].  Otherwise one scale per (row, block):
 * permute != 0 -> [ceil(rows/128)][nblocks][128], else [rows][nblocks]. */
void fluxref_quant_rows(const uint16_t *x, int64_t rows, int64_t cols, int32_t block_cols, float eps,
                        uint8_t *q, float *scale_inv, int32_t permute) {
  int64_t bc = block_cols == 0 ? cols : block_cols;
  int64_t nblocks = bc == 0 ? 0 : (cols + bc - 1) / bc;
  for (int64_t r = 0; r < rows; ++r) {
    for (int64_t b = 0; b < nblocks; ++b) {
      int64_t c0 = b * bc, c1 = c0 + bc < cols ? c0 + bc : cols;
      float amax = 0.f;
      for (int64_t c = c0; c < c1; ++c) amax = max_ignore_nan(amax, fabsf(bf16_to_f32(x[r * cols + c])));
      float scale = fluxref_compute_scale(amax, eps);
      float inv = (float)(1.0 / (double)scale);
      if (block_cols == 0) scale_inv[r] = inv;
      else if (permute) scale_inv[(r / 128) * (nblocks * 128) + b * 128 + (r % 128)] = inv;
      else scale_inv[r * nblocks + b] = inv;
      for (int64_t c = c0; c < c1; ++c) {
        float v = bf16_to_f32(x[r * cols + c]) * scale;
        q[r * cols + c] = fluxref_f32_to_e4m3(v);
      }
    }
  }
}

/* One scale per 128 x 128 block, taken over the part of the block inside the matrix;
 * scale_inv[ceil(rows/128)][ceil(cols/128)]. */
void fluxref_quant_square(const uint16_t *x, int64_t rows, int64_t cols, float eps, uint8_t *q,
                          float *scale_inv) {
  int64_t nby = (rows + 127) / 128, nbx = (cols + 127) / 128;
  for (int64_t by = 0; by < nby; ++by) {
    for (int64_t bx = 0; bx < nbx; ++bx) {
      int64_t r1 = by * 128 + 128 < rows ? by * 128 + 128 : rows;
      int64_t c1 = bx * 128 + 128 < cols ? bx * 128 + 128 : cols;
      float amax = 0.f;
      for (int64_t r = by * 128; r < r1; ++r)
        for (int64_t c = bx * 128; c < c1; ++c) amax = max_ignore_nan(amax, fabsf(bf16_to_f32(x[r * cols + c])));
      float scale = fluxref_compute_scale(amax, eps);
      scale_inv[by * nbx + bx] = 1.0f / scale;
      for (int64_t r = by * 128; r < r1; ++r)
        for (int64_t c = bx * 128; c < c1; ++c) q[r * cols + c] = fluxref_f32_to_e4m3(bf16_to_f32(x[r * cols + c]) * scale);
    }
  }
}
