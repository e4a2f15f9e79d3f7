// Declarations of the operator classes and free functions bound in pybind.cc.
#pragma once
#include "ths_common.h"

namespace flux_amd {

class GemmGroupedV3AGScatter {
 public:
  GemmGroupedV3AGScatter(DistEnvTPWithEP tp_env, MoeArguments moe_args);
  void clear_buffers();
  torch::Tensor forward(torch::Tensor inputs_shard, torch::Tensor weights, torch::Tensor splits_gpu,
                        torch::Tensor scatter_index, std::optional<torch::Tensor> output_scale,
                        std::optional<torch::Tensor> outputs_buf, std::optional<torch::Tensor> allgather_output,
                        bool fast_accum, int64_t sm_margin);
  std::vector<torch::Tensor> forward_multiple_weights(
      torch::Tensor inputs_shard, std::vector<torch::Tensor> weights, torch::Tensor splits_gpu,
      torch::Tensor scatter_index, std::optional<std::vector<torch::Tensor>> output_scale,
      std::optional<std::vector<torch::Tensor>> outputs_buf, std::optional<torch::Tensor> allgather_output,
      bool fast_accum, int64_t sm_margin);
  // forward() under every tile schedule, timed; the fastest is registered for the shape and recorded in
  // prof_ctx (gemm_grouped_v3_ag_scatter.cc:520-612).
  torch::Tensor profiling(torch::Tensor inputs_shard, torch::Tensor weights, torch::Tensor splits_gpu,
                          torch::Tensor scatter_index, std::optional<torch::Tensor> output_scale,
                          std::optional<torch::Tensor> outputs_buf, std::optional<torch::Tensor> allgather_output,
                          bool fast_accum, int64_t sm_margin, std::shared_ptr<ProfilingContext> prof_ctx);

 private:
  std::vector<torch::Tensor> forward_impl(torch::Tensor inputs_shard, std::vector<torch::Tensor> weights,
                                          torch::Tensor splits_gpu, torch::Tensor scatter_index,
                                          std::optional<std::vector<torch::Tensor>> output_scale,
                                          std::optional<std::vector<torch::Tensor>> outputs_buf,
                                          std::optional<torch::Tensor> allgather_output, bool fast_accum,
                                          int64_t sm_margin);
  DistEnvTPWithEP tp_env_;
  MoeArguments moe_args_;
  torch::Tensor gather_index_;
};

class GemmGroupedV3GatherRS {
 public:
  GemmGroupedV3GatherRS(int64_t total_num_experts, int64_t max_m, int64_t n_dim, int64_t topk, int64_t rank,
                        int64_t world_size, int64_t tp_world_size, int64_t ep_world_size,
                        int64_t max_input_groups, bool ep_in_dp);
  torch::Tensor forward_gather_rs(torch::Tensor input, torch::Tensor weight, torch::Tensor splits_cpu,
                                  torch::Tensor routing_idx, std::optional<torch::Tensor> n_tokens_per_rank,
                                  std::optional<torch::Tensor> input_scale,
                                  std::optional<torch::Tensor> weight_scale,
                                  std::optional<torch::Tensor> output_vec_scale, bool fast_accum,
                                  int64_t sm_margin, bool with_stream_sync);
  torch::Tensor forward_gather_rs_multiple(std::vector<torch::Tensor> inputs, std::vector<torch::Tensor> weights,
                                           torch::Tensor splits_cpu, torch::Tensor routing_idx,
                                           std::optional<torch::Tensor> n_tokens_per_rank,
                                           std::optional<std::vector<torch::Tensor>> input_scale,
                                           std::optional<std::vector<torch::Tensor>> weight_scale,
                                           std::optional<std::vector<torch::Tensor>> output_vec_scale,
                                           bool fast_accum, int64_t sm_margin, bool with_stream_sync);
  void ep_zero_buffer() {}  // expert-parallel scratch does not exist at world size 1
  // forward_gather_rs() under every tile schedule, timed; the fastest is registered for the shape and
  // recorded in prof_ctx (gemm_grouped_v3_gather_rs.cc:903-1000).
  torch::Tensor profiling(torch::Tensor input, torch::Tensor weight, torch::Tensor splits_cpu,
                          torch::Tensor routing_idx, std::optional<torch::Tensor> n_tokens_per_rank,
                          std::optional<torch::Tensor> input_scale, std::optional<torch::Tensor> weight_scale,
                          std::optional<torch::Tensor> output_vec_scale, bool fast_accum, int64_t sm_margin,
                          bool with_stream_sync, std::shared_ptr<ProfilingContext> prof_ctx);

 private:
  torch::Tensor forward_impl(std::vector<torch::Tensor> inputs, std::vector<torch::Tensor> weights,
                             torch::Tensor splits_cpu, torch::Tensor routing_idx,
                             std::optional<std::vector<torch::Tensor>> input_scale,
                             std::optional<std::vector<torch::Tensor>> weight_scale,
                             std::optional<std::vector<torch::Tensor>> output_vec_scale, bool with_stream_sync,
                             int64_t sm_margin);
  void lazy_init(const torch::Tensor &like);
  int64_t num_experts_, max_m_, n_dim_, topk_, max_input_groups_;
  bool inter_fp32_ = true;

 public:
  // Dtype of the intermediate between the GEMM and the reduction: fp32 (one rounding in the layer) or the 16-bit
  // output type (the reference's inter_D).  Only before the first forward: the buffers are allocated lazily.
  void set_intermediate_fp32(bool fp32) {
    TORCH_CHECK(inter_.empty(), "the intermediate's dtype is fixed once the op has run");
    inter_fp32_ = fp32;
  }

 private:
  int fused_mode_ = 0;  // 0: by shape, 1: always the fused epilogue reduce, 2: always GEMM + gather-reduce
  std::vector<torch::Tensor> inter_;
  torch::Tensor splits_dev_;
  torch::Tensor token_of_row_;  // inverse of routing_idx (the token of each sorted row), for the fused reduce
};

class GemmGroupedV3 {
 public:
  GemmGroupedV3(torch::Tensor weight, int64_t num_experts);
  torch::Tensor forward(torch::Tensor input, torch::Tensor splits_cpu);

 private:
  torch::Tensor weight_;
};

// Block-scaled fp8 GEMM of the reference (src/comm_none/ths_op/blockscale_gemm.h:24-94): the forward
// products, dense and grouped (forward_multistream is the same single launch).  The wgrad* methods (training-time
// weight gradients) are not on this path and are not built.
class BlockScaleGemm {
 public:
  BlockScaleGemm(at::ScalarType input_dtype, at::ScalarType weight_dtype, at::ScalarType output_dtype,
                 int32_t num_streams);
  // input [M, K] e4m3, weight [N, K] e4m3, input_scale [ceil(M/128), K/128, 128] (what
  // Quantization::quantize_vector_blockwise returns), weight_scale [ceil(N/128), K/128].
  torch::Tensor forward(torch::Tensor input, torch::Tensor weight, std::optional<torch::Tensor> bias,
                        std::optional<torch::Tensor> output, std::optional<torch::Tensor> input_scale,
                        std::optional<torch::Tensor> weight_scale);
  // input [M, K] sorted by expert, input_splits host [E], weight [E, N, K].  Scales either in the reference's
  // operand layouts (1-D tensors: per expert [K/128, M_e] back to back; per expert [K/128, N/128]:
  // blockscale_gemm.cc:703-722) or as the quantisation ops return them (3-D tensors: input_scale
  // [ceil(M/128), K/128, 128] over the sorted rows, weight_scale [E, N/128, K/128]).
  torch::Tensor forward_grouped(torch::Tensor input, torch::Tensor input_splits, torch::Tensor weight,
                                std::optional<torch::Tensor> bias, std::optional<torch::Tensor> output,
                                torch::Tensor input_scale, torch::Tensor weight_scale);
  // The grouped product with input_scale as [M, K/128] (any strides) and weight_scale [E, N/128, K/128]: the
  // arguments of the reference's multi-stream form; one launch here.
  torch::Tensor forward_multistream(torch::Tensor input, torch::Tensor input_splits, torch::Tensor weight,
                                    std::optional<torch::Tensor> bias, std::optional<torch::Tensor> output,
                                    std::optional<torch::Tensor> input_scale, std::optional<torch::Tensor> weight_scale);
  torch::Tensor reference(torch::Tensor input, torch::Tensor weight, std::optional<torch::Tensor> bias,
                          std::optional<torch::Tensor> output, std::optional<torch::Tensor> input_scale,
                          std::optional<torch::Tensor> weight_scale, bool is_groupwise_b);
  torch::Tensor profiling(torch::Tensor input, torch::Tensor weight, std::optional<torch::Tensor> bias,
                          std::optional<torch::Tensor> output, std::optional<torch::Tensor> input_scale,
                          std::optional<torch::Tensor> weight_scale, std::shared_ptr<ProfilingContext> prof_ctx);

 private:
  at::ScalarType input_dtype_, weight_dtype_, output_dtype_;
};

class Quantization {
 public:
  using Result = std::tuple<torch::Tensor, torch::Tensor, std::optional<torch::Tensor>, std::optional<torch::Tensor>>;
  Quantization(at::ScalarType input_dtype, at::ScalarType output_dtype, int32_t num_streams);
  Result quantize_vector_blockwise(torch::Tensor input, bool return_transpose, float eps);
  Result quantize_square_blockwise(torch::Tensor input, bool return_transpose, float eps);
  Result batch_quantize_square_blockwise(torch::Tensor input, bool return_transpose, float eps);
  std::tuple<torch::Tensor, torch::Tensor> quantize_rowwise(torch::Tensor input, float eps);

 private:
  at::ScalarType input_dtype_, output_dtype_;
};

torch::Tensor calc_scatter_index(torch::Tensor choosed_experts, torch::Tensor splits);
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor> moe_route_sort(torch::Tensor choosed_experts,
                                                                                      int64_t nexperts);
torch::Tensor topk_scatter_reduce(std::vector<torch::Tensor> inputs, torch::Tensor scatter_idx, int64_t topk);
torch::Tensor topk_weighted_gather_reduce(std::vector<torch::Tensor> inputs, torch::Tensor routing_idx,
                                          int64_t topk, std::optional<torch::Tensor> row_weight, double scale);
bool bitwise_check(torch::Tensor a, torch::Tensor b);

}  // namespace flux_amd
