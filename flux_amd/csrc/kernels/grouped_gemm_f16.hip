// fp16 instantiation of the grouped GEMM MFMA kernel: the 2-byte kernel with v_mfma_f32_16x16x32_f16 and an fp16
// output cast.
#define FLUXMI_HALF_IS_F16 1
#include "grouped_gemm_kernel.hpp"

namespace fluxmi {
int launch_grouped_gemm_f16(const GemmParams &p, int grid, hipStream_t s) { return launch_mfma<2>(p, grid, s); }
}  // namespace fluxmi
