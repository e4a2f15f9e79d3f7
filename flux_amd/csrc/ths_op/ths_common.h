// Host-side glue shared by the torch ops: argument checks in the style of the reference's
// CHECK_INPUT / CHECK_NDIM (include/flux/ths_op/util.h:24-47), the current HIP stream, and conversion
// of a C-ABI status into the exception type the reference raises (std::runtime_error -> RuntimeError).
#pragma once
#include <c10/hip/HIPStream.h>
#include <torch/extension.h>

#include <optional>
#include <stdexcept>
#include <string>
#include <vector>

#include "fluxmi.h"
#include "tuning.h"

namespace flux_amd {

inline void *current_stream() { return static_cast<void *>(c10::hip::getCurrentHIPStream().stream()); }

inline void check_status(int status, const char *what) {
  if (status != FLUXMI_OK) {
    throw std::runtime_error(std::string(what) + " failed (" + std::to_string(status) + "): " +
                             fluxmi_last_error());
  }
}

inline bool is_fp8(at::ScalarType t) { return t == at::ScalarType::Float8_e4m3fn; }

inline int32_t to_fluxmi_dtype(at::ScalarType t) {
  if (t == at::ScalarType::BFloat16) return FLUXMI_BF16;
  if (t == at::ScalarType::Float8_e4m3fn) return FLUXMI_FP8_E4M3;
  if (t == at::ScalarType::Half) return FLUXMI_FP16;
  TORCH_CHECK(false, "flux_amd: unsupported dtype ", t, " (bf16, fp16 and float8_e4m3fn are built)");
  return -1;
}

// Output dtype of the two MoE ops for an operand dtype: fp16 in gives fp16 out, bf16 and fp8 in give bf16 out
// (test/python/moe_ag_scatter/test_moe_ag.py:424-430 OUT_DTYPE_MAP; gemm_grouped_v3_gather_rs.cc:53-63).
inline at::ScalarType moe_output_dtype(at::ScalarType in) {
  return in == at::ScalarType::Half ? at::ScalarType::Half : at::ScalarType::BFloat16;
}

#define FLUX_AMD_CHECK_INPUT(x, st)                                                        \
  do {                                                                                     \
    TORCH_CHECK((x).is_cuda(), #x " must be a device tensor");                              \
    TORCH_CHECK((x).is_contiguous(), #x " must be contiguous");                             \
    TORCH_CHECK((x).scalar_type() == (st), "Inconsistency of Tensor type: " #x " is ",      \
                (x).scalar_type(), ", expected ", (st));                                    \
  } while (0)

#define FLUX_AMD_CHECK_NDIM(x, n) TORCH_CHECK((x).dim() == (n), #x " must have ", (n), " dimensions, got ", (x).dim())

#define FLUX_AMD_CHECK_2D(x, d0, d1)                                                                \
  TORCH_CHECK((x).dim() == 2 && (x).size(0) == (d0) && (x).size(1) == (d1), #x " shape mismatch: ", \
              (x).sizes(), " expected [", (d0), ", ", (d1), "]")

#define FLUX_AMD_CHECK_3D(x, d0, d1, d2)                                                              \
  TORCH_CHECK((x).dim() == 3 && (x).size(0) == (d0) && (x).size(1) == (d1) && (x).size(2) == (d2),    \
              #x " shape mismatch: ", (x).sizes(), " expected [", (d0), ", ", (d1), ", ", (d2), "]")

// Small value types of the reference's op surface.
struct MoeArguments {  // src/ths_op/ths_op.cc + src/pybind/ths_op.cc:121-146
  int32_t max_ntokens, hidden, ffn_hidden, nexperts, topk;
  at::ScalarType input_dtype, output_dtype;
};

struct DistEnvTPWithEP {  // include/flux/ths_op/ths_op.h:117-130; only world size 1 exists here
  int32_t rank = 0, world_size = 1, nnodes = 1, ep_rank = 0, ep_size = 1, ffn_tp_size = 1, ffn_tp_rank = 0;
  std::string to_string() const {
    return "DistEnvTPWithEP(rank=0,world_size=1,nnodes=1,ep_rank=0,ep_size=1)";
  }
};

// Filled grouped-GEMM argument block (everything on the current stream).
void run_grouped_gemm(const torch::Tensor &a, const torch::Tensor &b, const torch::Tensor &splits_dev,
                      torch::Tensor &d, const int32_t *gather_a, int64_t max_rows, const float *alpha,
                      const float *row_scale, const float *col_scale, const float *scalar_dev, int64_t sm_margin);

// Launch tuning of a grouped GEMM: CUs to leave free (Flux's sm_margin) and the tile schedule registered
// for the problem's shape, if any.
void apply_launch_tuning(fluxmi_grouped_gemm_args &args, int32_t ngroups, int64_t sm_margin);

}  // namespace flux_amd
