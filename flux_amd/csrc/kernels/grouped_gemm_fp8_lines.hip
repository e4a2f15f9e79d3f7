// fp8 (e4m3) instantiation of the grouped GEMM MFMA kernel with whole-line ring fills.
#define FLUXMI_LINE_FILLS 1
#include "grouped_gemm_kernel.hpp"

namespace fluxmi {
int launch_grouped_gemm_fp8_lines(const GemmParams &p, int grid, hipStream_t s) { return launch_mfma<1>(p, grid, s); }
}  // namespace fluxmi
