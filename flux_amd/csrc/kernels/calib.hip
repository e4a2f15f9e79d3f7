// Calibration streams: what the memory system of the GPU at hand gives a kernel that only streams.  A read stream
// (every byte of a buffer read once, 16 bytes per lane and load, eight loads in flight per lane, a few bytes
// written per workgroup) and a copy (the same reads, each stored again).  The benchmark times them beside the
// HBM-bound kernels of the path (top-k gather-reduce, quantisation) so that their fraction of the published
// bandwidth can be read against what a plain stream reaches on the same machine, and the copy's known traffic
// scales the byte counters of the profiler.
#include "common.hpp"

namespace fluxmi {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
constexpr int kCalibThreads = 256;
constexpr int kCalibUnroll = 8;

template <bool COPY>
__global__ __launch_bounds__(kCalibThreads) void calib_stream_kernel(const u32x4 *__restrict__ src, u32x4 *__restrict__ dst,
                                                                      size_t nvec) {
  const size_t chunk = static_cast<size_t>(kCalibThreads) * kCalibUnroll;
  u32x4 acc = {0u, 0u, 0u, 0u};
  for (size_t base = static_cast<size_t>(blockIdx.x) * chunk; base < nvec; base += static_cast<size_t>(gridDim.x) * chunk) {
    u32x4 v[kCalibUnroll];
#pragma unroll
    for (int u = 0; u < kCalibUnroll; ++u) {
      const size_t i = base + static_cast<size_t>(u) * kCalibThreads + threadIdx.x;
      v[u] = i < nvec ? __builtin_nontemporal_load(src + i) : u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int u = 0; u < kCalibUnroll; ++u) {
      const size_t i = base + static_cast<size_t>(u) * kCalibThreads + threadIdx.x;
      if constexpr (COPY) {
        if (i < nvec) __builtin_nontemporal_store(v[u], dst + i);
      } else {
        acc ^= v[u];
      }
    }
  }
  if constexpr (!COPY) {
    // One vector per lane of the first wave of every workgroup keeps the loads alive (the xor of everything read).
    if (threadIdx.x < 64) dst[static_cast<size_t>(blockIdx.x) * 64 + threadIdx.x] = acc;
    else if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u) dst[static_cast<size_t>(blockIdx.x) * 64] = acc;
  }
}

}  // namespace
}  // namespace fluxmi

extern "C" size_t fluxmi_calib_stream_sink_bytes(void) {
  const int cus = fluxmi_device_cu_count();
  return static_cast<size_t>(cus > 0 ? cus : 256) * 8 * 64 * 16;
}

extern "C" int fluxmi_calib_stream(const void *src, void *dst, size_t bytes, int32_t copy, void *stream) {
  using namespace fluxmi;
  FLUXMI_REQUIRE(src != nullptr && dst != nullptr, FLUXMI_ERR_INVALID_ARG, "calib_stream: null pointer");
  FLUXMI_REQUIRE(bytes % 16 == 0 && aligned16(src) && aligned16(dst), FLUXMI_ERR_INVALID_ARG,
                 "calib_stream: bytes and pointers must be multiples of 16");
  if (bytes == 0) return FLUXMI_OK;
  const int cus = fluxmi_device_cu_count();
  FLUXMI_REQUIRE(cus > 0, FLUXMI_ERR_HIP, "calib_stream: cannot query the device");
  const size_t nvec = bytes / 16;
  const size_t chunk = static_cast<size_t>(kCalibThreads) * kCalibUnroll;
  const size_t want = (nvec + chunk - 1) / chunk;
  const unsigned grid = static_cast<unsigned>(want < static_cast<size_t>(cus) * 8 ? want : static_cast<size_t>(cus) * 8);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (copy) hipLaunchKernelGGL(calib_stream_kernel<true>, dim3(grid), dim3(kCalibThreads), 0, s, static_cast<const u32x4 *>(src),
                               static_cast<u32x4 *>(dst), nvec);
  else hipLaunchKernelGGL(calib_stream_kernel<false>, dim3(grid), dim3(kCalibThreads), 0, s, static_cast<const u32x4 *>(src),
                          static_cast<u32x4 *>(dst), nvec);
  FLUXMI_HIP_CHECK(hipGetLastError());
  return FLUXMI_OK;
}
