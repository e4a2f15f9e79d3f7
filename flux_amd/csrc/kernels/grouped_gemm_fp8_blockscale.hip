// Block-scaled fp8 (e4m3) instantiation of the grouped GEMM MFMA kernel: 256 x 128 tiles, promotion every 128 of K.
#include "grouped_gemm_kernel.hpp"

namespace fluxmi {
int launch_grouped_gemm_fp8_blockscale(const GemmParams &p, int grid, hipStream_t s) {
  return launch_mfma<1, true>(p, grid, s);
}
}  // namespace fluxmi
