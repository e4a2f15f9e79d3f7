/* The C-ABI of include/fluxmi.h driven from plain C with the HIP runtime and nothing else (no torch, no
 * Python): what a C or C++ host that links libfluxmi_kernels.so does.  Runs the four kernels of the path on
 * small inputs and checks them against loops written here.  Built by flux_amd/build.py into
 * flux_amd/lib/capi_smoke and run by tests/test_gpu_capi_c.py; exit status 0 = every check passed. */
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "fluxmi.h"

#define HIP_OK(expr)                                                                     \
  do {                                                                                   \
    hipError_t e_ = (expr);                                                              \
    if (e_ != hipSuccess) {                                                              \
      fprintf(stderr, "%s failed: %s\n", #expr, hipGetErrorString(e_));                  \
      return 2;                                                                          \
    }                                                                                    \
  } while (0)

#define FLUX_OK(expr)                                                                    \
  do {                                                                                   \
    int rc_ = (expr);                                                                    \
    if (rc_ != FLUXMI_OK) {                                                              \
      fprintf(stderr, "%s returned %d: %s\n", #expr, rc_, fluxmi_last_error());          \
      return 3;                                                                          \
    }                                                                                    \
  } while (0)

static uint16_t f2bf(float f) { /* round to nearest even */
  uint32_t u;
  memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
static float bf2f(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static uint32_t lcg(uint32_t *s) { return *s = *s * 1664525u + 1013904223u; }
static float unit(uint32_t *s) { return (float)(lcg(s) >> 8) / 16777216.0f - 0.5f; } /* [-0.5, 0.5) */

enum { T = 96, TOPK = 2, E = 4, M = T * TOPK, H = 64, N = 72 };

int main(void) {
  uint32_t seed = 12345u;
  static int32_t choosed[M], splits[E], offsets[E + 1], scatter[M], gather[M], tki[M];
  static int32_t want_scatter[M], want_splits[E];
  for (int t = 0; t < T; ++t) { /* two distinct experts per token */
    const int a = (int)(lcg(&seed) >> 10) % E, b = (a + 1 + (int)(lcg(&seed) >> 10) % (E - 1)) % E;
    choosed[2 * t] = a;
    choosed[2 * t + 1] = b;
  }
  memset(want_splits, 0, sizeof want_splits);
  for (int i = 0; i < M; ++i) ++want_splits[choosed[i]];
  {
    int off[E], acc = 0;
    for (int e = 0; e < E; ++e) off[e] = acc, acc += want_splits[e];
    for (int i = 0; i < M; ++i) want_scatter[i] = off[choosed[i]]++;
  }

  /* ---- routing ------------------------------------------------------------------------------ */
  int32_t *d_choosed, *d_splits, *d_offsets, *d_scatter, *d_gather, *d_tki;
  void *d_ws;
  const size_t ws_bytes = fluxmi_moe_route_sort_workspace_bytes(T, TOPK, E);
  HIP_OK(hipMalloc((void **)&d_choosed, sizeof choosed));
  HIP_OK(hipMalloc((void **)&d_splits, sizeof splits));
  HIP_OK(hipMalloc((void **)&d_offsets, sizeof offsets));
  HIP_OK(hipMalloc((void **)&d_scatter, sizeof scatter));
  HIP_OK(hipMalloc((void **)&d_gather, sizeof gather));
  HIP_OK(hipMalloc((void **)&d_tki, sizeof tki));
  HIP_OK(hipMalloc(&d_ws, ws_bytes ? ws_bytes : 16));
  HIP_OK(hipMemcpy(d_choosed, choosed, sizeof choosed, hipMemcpyHostToDevice));
  FLUX_OK(fluxmi_moe_route_sort(d_choosed, T, TOPK, E, d_splits, d_offsets, d_scatter, d_gather, d_tki, d_ws, ws_bytes,
                                NULL));
  HIP_OK(hipDeviceSynchronize());
  HIP_OK(hipMemcpy(splits, d_splits, sizeof splits, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(offsets, d_offsets, sizeof offsets, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(scatter, d_scatter, sizeof scatter, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(gather, d_gather, sizeof gather, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(tki, d_tki, sizeof tki, hipMemcpyDeviceToHost));
  if (memcmp(splits, want_splits, sizeof splits) || memcmp(scatter, want_scatter, sizeof scatter) || offsets[E] != M) {
    fprintf(stderr, "routing: splits / scatter_index differ from the stable counting sort\n");
    return 1;
  }
  for (int i = 0; i < M; ++i)
    if (gather[scatter[i]] != i / TOPK || tki[scatter[i]] != i % TOPK) {
      fprintf(stderr, "routing: gather_index / topk_index are not the inverse permutation at %d\n", i);
      return 1;
    }
  /* the same sort over the library's static scratch array: the entry point that allocates nothing */
  {
    static int32_t scatter2[M], gather2[M], splits2[E];
    HIP_OK(hipMemset(d_scatter, 0xff, sizeof scatter));
    HIP_OK(hipMemset(d_gather, 0xff, sizeof gather));
    HIP_OK(hipMemset(d_splits, 0xff, sizeof splits));
    FLUX_OK(fluxmi_moe_route_sort_static(d_choosed, T, TOPK, E, d_splits, d_offsets, d_scatter, d_gather, d_tki, NULL));
    HIP_OK(hipDeviceSynchronize());
    HIP_OK(hipMemcpy(splits2, d_splits, sizeof splits2, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(scatter2, d_scatter, sizeof scatter2, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(gather2, d_gather, sizeof gather2, hipMemcpyDeviceToHost));
    if (memcmp(splits2, splits, sizeof splits) || memcmp(scatter2, scatter, sizeof scatter) ||
        memcmp(gather2, gather, sizeof gather) || fluxmi_moe_route_sort_static_max_bytes() < ws_bytes) {
      fprintf(stderr, "routing: the static-scratch sort differs from the workspace sort\n");
      return 1;
    }
  }
  printf("routing ok\n");

  /* ---- layer0: gather + grouped GEMM, bf16 ------------------------------------------------------ */
  static uint16_t x[T * H], w[E * N * H], y[M * N];
  for (int i = 0; i < T * H; ++i) x[i] = f2bf(unit(&seed) * 2.f);
  for (int i = 0; i < E * N * H; ++i) w[i] = f2bf(unit(&seed) * 0.25f);
  uint16_t *d_x, *d_w, *d_y;
  HIP_OK(hipMalloc((void **)&d_x, sizeof x));
  HIP_OK(hipMalloc((void **)&d_w, sizeof w));
  HIP_OK(hipMalloc((void **)&d_y, sizeof y));
  HIP_OK(hipMemcpy(d_x, x, sizeof x, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_w, w, sizeof w, hipMemcpyHostToDevice));
  fluxmi_grouped_gemm_args ga;
  memset(&ga, 0, sizeof ga);
  ga.dtype = FLUXMI_BF16;
  ga.nexperts = E;
  ga.max_rows = M;
  ga.n = N;
  ga.k = H;
  ga.a_rows = T;
  ga.a = d_x;
  ga.b = d_w;
  ga.d = d_y;
  ga.splits = d_splits;
  ga.gather_a = d_gather;
  ga.scalar_scale = 1.0f;
  if (fluxmi_grouped_gemm_kernel_kind(&ga) != 1) {
    fprintf(stderr, "grouped GEMM: K = %d bf16 (rows of %d bytes) must take the MFMA kernel\n", H, 2 * H);
    return 1;
  }
  FLUX_OK(fluxmi_grouped_gemm(&ga, NULL, 0, NULL));
  HIP_OK(hipDeviceSynchronize());
  HIP_OK(hipMemcpy(y, d_y, sizeof y, hipMemcpyDeviceToHost));
  for (int r = 0; r < M; ++r) {
    int e = 0;
    while (r >= offsets[e] + splits[e]) ++e;
    for (int n = 0; n < N; ++n) {
      float acc = 0.f;
      for (int k = 0; k < H; ++k) acc += bf2f(x[gather[r] * H + k]) * bf2f(w[(e * N + n) * H + k]);
      if (fabsf(bf2f(y[r * N + n]) - acc) > 1e-2f + 1e-2f * fabsf(acc)) {
        fprintf(stderr, "grouped GEMM: row %d col %d got %g want %g\n", r, n, bf2f(y[r * N + n]), acc);
        return 1;
      }
    }
  }
  printf("grouped gemm ok\n");

  /* ---- top-k gather-reduce back to token order -------------------------------------------------- */
  static float row_w[M];
  static uint16_t out[T * N];
  for (int i = 0; i < M; ++i) row_w[i] = 0.25f + (float)(lcg(&seed) >> 8) / 33554432.0f;
  float *d_row_w;
  uint16_t *d_out;
  HIP_OK(hipMalloc((void **)&d_row_w, sizeof row_w));
  HIP_OK(hipMalloc((void **)&d_out, sizeof out));
  HIP_OK(hipMemcpy(d_row_w, row_w, sizeof row_w, hipMemcpyHostToDevice));
  const void *groups[1] = {d_y};
  FLUX_OK(fluxmi_topk_gather_reduce(groups, 1, 0, d_scatter, d_row_w, 1.0f, T, TOPK, N, d_out, NULL));
  HIP_OK(hipDeviceSynchronize());
  HIP_OK(hipMemcpy(out, d_out, sizeof out, hipMemcpyDeviceToHost));
  for (int t = 0; t < T; ++t)
    for (int n = 0; n < N; ++n) {
      float acc = 0.f;
      for (int j = 0; j < TOPK; ++j) {
        const int r = scatter[t * TOPK + j];
        acc = fmaf(row_w[r], bf2f(y[r * N + n]), acc);
      }
      if (f2bf(acc) != out[t * N + n]) {
        fprintf(stderr, "gather-reduce: token %d col %d got %g want %g\n", t, n, bf2f(out[t * N + n]), acc);
        return 1;
      }
    }
  printf("gather-reduce ok\n");

  /* ---- the same layer with the reduction in the GEMM's epilogue: out2[t] = sum_j w[r_j] * (x[t] @ W[e_j]^T) ---- */
  {
    static uint16_t out2[T * N];
    uint16_t *d_out2;
    void *d_acc;
    const size_t acc_bytes = fluxmi_grouped_gemm_topk_reduce_workspace_bytes(T, N);
    HIP_OK(hipMalloc((void **)&d_out2, sizeof out2));
    HIP_OK(hipMalloc(&d_acc, acc_bytes));
    fluxmi_grouped_gemm_args fa = ga;
    fa.d = NULL;
    fa.row_scale = d_row_w;
    FLUX_OK(fluxmi_grouped_gemm_topk_reduce(&fa, d_gather, T, d_out2, d_acc, acc_bytes, NULL));
    HIP_OK(hipDeviceSynchronize());
    HIP_OK(hipMemcpy(out2, d_out2, sizeof out2, hipMemcpyDeviceToHost));
    for (int t = 0; t < T; ++t)
      for (int n = 0; n < N; ++n) {
        float want = 0.f;
        for (int j = 0; j < TOPK; ++j) {
          const int r = scatter[t * TOPK + j];
          int e = 0;
          while (r >= offsets[e] + splits[e]) ++e;
          float acc = 0.f;
          for (int k = 0; k < H; ++k) acc += bf2f(x[t * H + k]) * bf2f(w[(e * N + n) * H + k]);
          want += row_w[r] * acc;
        }
        if (fabsf(bf2f(out2[t * N + n]) - want) > 1e-2f + 1e-2f * fabsf(want)) {
          fprintf(stderr, "fused reduce: token %d col %d got %g want %g\n", t, n, bf2f(out2[t * N + n]), want);
          return 1;
        }
      }
    printf("fused epilogue reduce ok\n");
  }

  /* ---- e4m3 quantisation per row: scale_inv = amax / 448, the row's largest element maps to +-448 ------- */
  static uint8_t q[T * H];
  static float sinv[T];
  uint8_t *d_q;
  float *d_sinv;
  HIP_OK(hipMalloc((void **)&d_q, sizeof q));
  HIP_OK(hipMalloc((void **)&d_sinv, sizeof sinv));
  FLUX_OK(fluxmi_quant_e4m3_rowwise(d_x, T, H, 0, 0.0f, d_q, d_sinv, 0, NULL));
  HIP_OK(hipDeviceSynchronize());
  HIP_OK(hipMemcpy(q, d_q, sizeof q, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(sinv, d_sinv, sizeof sinv, hipMemcpyDeviceToHost));
  for (int t = 0; t < T; ++t) {
    float amax = 0.f;
    int arg = 0;
    for (int k = 0; k < H; ++k)
      if (fabsf(bf2f(x[t * H + k])) > amax) amax = fabsf(bf2f(x[t * H + k])), arg = k;
    const float scale = 448.0f / amax;
    const float want = (float)(1.0 / (double)scale);
    if (sinv[t] != want || (q[t * H + arg] & 0x7f) != 0x7e) { /* 0x7e = 448, the largest finite e4m3 */
      fprintf(stderr, "quant: row %d scale_inv %g want %g, code of the row maximum 0x%02x\n", t, sinv[t], want,
              q[t * H + arg]);
      return 1;
    }
  }
  printf("quant ok\n");

  /* ---- error reporting --------------------------------------------------------------------------- */
  ga.dtype = 99;
  if (fluxmi_grouped_gemm(&ga, NULL, 0, NULL) != FLUXMI_ERR_INVALID_ARG || strstr(fluxmi_last_error(), "dtype") == NULL) {
    fprintf(stderr, "error path: expected FLUXMI_ERR_INVALID_ARG naming the dtype\n");
    return 1;
  }
  printf("capi_smoke: all checks passed (version %d, %d CUs)\n", fluxmi_version(), fluxmi_device_cu_count());
  return 0;
}
