// Shared host/device helpers for the gfx950 kernels: error reporting for the C-ABI, wave64 primitives.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <cstdarg>
#include <cstdio>

#include "fluxmi.h"

namespace fluxmi {

// Thread-local message returned by fluxmi_last_error(); defined in api.hip.
void set_error(const char *fmt, ...);

#define FLUXMI_REQUIRE(cond, status, ...)   \
  do {                                      \
    if (!(cond)) {                          \
      ::fluxmi::set_error(__VA_ARGS__);     \
      return (status);                      \
    }                                       \
  } while (0)

#define FLUXMI_HIP_CHECK(expr)                                                            \
  do {                                                                                    \
    hipError_t _e = (expr);                                                               \
    if (_e != hipSuccess) {                                                               \
      ::fluxmi::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__, \
                          __LINE__);                                                      \
      return FLUXMI_ERR_HIP;                                                              \
    }                                                                                     \
  } while (0)

// Raises the dynamic-LDS limit of `kernel` to `bytes` once per device (the attribute lives with the
// device's copy of the code object).  `done_mask` is a function-local static of the caller, one bit per
// device id; a lost race only repeats the idempotent call.
inline int ensure_dynamic_lds(const void *kernel, int bytes, std::atomic<uint64_t> &done_mask) {
  int dev = 0;
  FLUXMI_HIP_CHECK(hipGetDevice(&dev));
  const uint64_t bit = uint64_t{1} << (dev & 63);
  if (done_mask.load(std::memory_order_acquire) & bit) return FLUXMI_OK;
  FLUXMI_HIP_CHECK(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
  done_mask.fetch_or(bit, std::memory_order_release);
  return FLUXMI_OK;
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

constexpr int kWave = 64;

// ---- wave64 primitives -------------------------------------------------------------------------
__device__ __forceinline__ int lane_id() {
  return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

// Number of set bits of `mask` strictly below the calling lane.
__device__ __forceinline__ int popc_below_lane(uint64_t mask) {
  return __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(mask >> 32),
                                   __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), 0u));
}

// Inclusive prefix sum across the 64 lanes of a wave.
__device__ __forceinline__ int wave_inclusive_scan(int v) {
  const int lane = lane_id();
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    int up = __shfl_up(v, off, 64);
    if (lane >= off) v += up;
  }
  return v;
}

__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) {
  return __uint_as_float(static_cast<uint32_t>(b) << 16);
}

__device__ __forceinline__ float f16_bits_to_float(uint16_t b) {
  return static_cast<float>(__builtin_bit_cast(_Float16, b));
}

// fp32 -> fp16 bits, round to nearest even (v_cvt_f16_f32).
__device__ __forceinline__ uint16_t float_to_f16_bits(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));
}

// fp32 -> bf16 bits, round to nearest even, NaN kept quiet.
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}

}  // namespace fluxmi
