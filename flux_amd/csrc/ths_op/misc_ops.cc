// Quantization (src/quantization/ths_op/quantization.{h,cc}) and the free functions of the reference's
// module on this path: calc_scatter_index (src/pybind/ths_op.cc:59-78), topk_scatter_reduce
// (src/moe_gather_rs/ths_op/topk_scatter_reduce.cc:30-56), bitwise_check (src/ths_op/ths_op.cc).
#include "ths_ops.h"

namespace flux_amd {

constexpr int64_t kBlock = 128;  // BLOCK_TILE_DIM of the reference's quantisation kernels

Quantization::Quantization(at::ScalarType input_dtype, at::ScalarType output_dtype, int32_t /*num_streams*/)
    : input_dtype_(input_dtype), output_dtype_(output_dtype) {
  // The reference hard-wires the same pair (src/quantization/quantization.cu:1399-1400).
  TORCH_CHECK(input_dtype == at::kBFloat16, "Quantization: input dtype must be bfloat16, got ", input_dtype);
  TORCH_CHECK(output_dtype == at::ScalarType::Float8_e4m3fn, "Quantization: output dtype must be float8_e4m3fn, got ",
              output_dtype);
}

static void quant_call(const torch::Tensor &x, int32_t block_cols, float eps, torch::Tensor &q,
                       torch::Tensor &scale_inv, bool permute) {
  check_status(fluxmi_quant_e4m3_rowwise(x.data_ptr(), x.size(0), x.size(1), block_cols, eps, q.data_ptr(),
                                         scale_inv.data_ptr<float>(), permute ? 1 : 0, current_stream()),
               "fluxmi_quant_e4m3_rowwise");
}

Quantization::Result Quantization::quantize_vector_blockwise(torch::Tensor input, bool return_transpose, float eps) {
  TORCH_CHECK(input.dim() == 2, "Input must have 2 dimensions.");
  FLUX_AMD_CHECK_INPUT(input, input_dtype_);
  const int64_t rows = input.size(0), cols = input.size(1);
  const int64_t bx = (cols + kBlock - 1) / kBlock, by = (rows + kBlock - 1) / kBlock;
  torch::Tensor out = torch::empty({rows, cols}, input.options().dtype(output_dtype_));
  // [ceil(M/128), ceil(K/128), 128] with the row inside its 128-row block fastest
  // (quantization.cc:91-93, quantization.cu:612-621).  Padding rows of the last block stay zero.
  // Entries of rows (columns) past the end of the last block are not written: zero-fill only when there are any.
  auto fopt = input.options().dtype(at::kFloat);
  torch::Tensor scale = rows % kBlock ? torch::zeros({by, bx, kBlock}, fopt) : torch::empty({by, bx, kBlock}, fopt);
  std::optional<torch::Tensor> out_t, scale_t;
  if (return_transpose) {
    // The transposed matrix with one scale per (column, 128-row block), from the same read of the input.
    out_t = torch::empty({cols, rows}, input.options().dtype(output_dtype_));
    scale_t = cols % kBlock ? torch::zeros({bx, by, kBlock}, fopt) : torch::empty({bx, by, kBlock}, fopt);
  }
  check_status(fluxmi_quant_e4m3_block128(input.data_ptr(), rows, cols, eps, out.data_ptr(), scale.data_ptr<float>(),
                                          return_transpose ? out_t->data_ptr() : nullptr,
                                          return_transpose ? scale_t->data_ptr<float>() : nullptr, current_stream()),
               "fluxmi_quant_e4m3_block128");
  return {out, scale, out_t, scale_t};
}

// One scale per 128 x 128 block; `input` is [batch, rows, cols] (quantization.cc:152-221 is batch = 1,
// :228-316 loops over the batch on side streams: here the batch is one launch on the current stream).
static Quantization::Result quant_square(const torch::Tensor &input, int64_t batch, int64_t rows, int64_t cols,
                                         bool batched, bool return_transpose, float eps, at::ScalarType out_dtype) {
  const int64_t bx = (cols + kBlock - 1) / kBlock, by = (rows + kBlock - 1) / kBlock;
  auto shape = [&](int64_t a, int64_t b) {
    return batched ? std::vector<int64_t>{batch, a, b} : std::vector<int64_t>{a, b};
  };
  torch::Tensor out = torch::empty(shape(rows, cols), input.options().dtype(out_dtype));
  torch::Tensor scale = torch::empty(shape(by, bx), input.options().dtype(at::kFloat));
  std::optional<torch::Tensor> out_t, scale_t;
  if (return_transpose) {
    out_t = torch::empty(shape(cols, rows), input.options().dtype(out_dtype));
    scale_t = torch::empty(shape(bx, by), input.options().dtype(at::kFloat));
  }
  check_status(fluxmi_quant_e4m3_square(input.data_ptr(), batch, rows, cols, eps, out.data_ptr(),
                                        scale.data_ptr<float>(), return_transpose ? out_t->data_ptr() : nullptr,
                                        return_transpose ? scale_t->data_ptr<float>() : nullptr, current_stream()),
               "fluxmi_quant_e4m3_square");
  return {out, scale, out_t, scale_t};
}

Quantization::Result Quantization::quantize_square_blockwise(torch::Tensor input, bool return_transpose, float eps) {
  TORCH_CHECK(input.dim() == 2, "Input must have 2 dimensions.");
  FLUX_AMD_CHECK_INPUT(input, input_dtype_);
  return quant_square(input, 1, input.size(0), input.size(1), false, return_transpose, eps, output_dtype_);
}

Quantization::Result Quantization::batch_quantize_square_blockwise(torch::Tensor input, bool return_transpose,
                                                                   float eps) {
  TORCH_CHECK(input.dim() == 3, "Input must have 3 dimensions.");
  FLUX_AMD_CHECK_INPUT(input, input_dtype_);
  return quant_square(input, input.size(0), input.size(1), input.size(2), true, return_transpose, eps,
                      output_dtype_);
}

std::tuple<torch::Tensor, torch::Tensor> Quantization::quantize_rowwise(torch::Tensor input, float eps) {
  TORCH_CHECK(input.dim() == 2, "Input must have 2 dimensions.");
  FLUX_AMD_CHECK_INPUT(input, input_dtype_);
  torch::Tensor out = torch::empty(input.sizes(), input.options().dtype(output_dtype_));
  torch::Tensor scale = torch::empty({input.size(0)}, input.options().dtype(at::kFloat));
  quant_call(input, 0, eps, out, scale, false);
  return {out, scale};
}

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor> moe_route_sort(torch::Tensor choosed_experts,
                                                                                      int64_t nexperts) {
  FLUX_AMD_CHECK_INPUT(choosed_experts, at::kInt);
  FLUX_AMD_CHECK_NDIM(choosed_experts, 2);
  const int32_t ntokens = static_cast<int32_t>(choosed_experts.size(0));
  const int32_t topk = static_cast<int32_t>(choosed_experts.size(1));
  TORCH_CHECK(topk >= 1, "topk must be positive");
  auto iopt = choosed_experts.options();
  torch::Tensor splits = torch::empty({nexperts}, iopt);
  torch::Tensor scatter = torch::empty_like(choosed_experts);
  torch::Tensor gather = torch::empty({static_cast<int64_t>(ntokens) * topk}, iopt);
  torch::Tensor topk_index = torch::empty({static_cast<int64_t>(ntokens) * topk}, iopt);
  const size_t ws_bytes = fluxmi_moe_route_sort_workspace_bytes(ntokens, topk, static_cast<int32_t>(nexperts));
  torch::Tensor ws = torch::empty({static_cast<int64_t>(ws_bytes > 0 ? ws_bytes : 1)}, iopt.dtype(at::kByte));
  check_status(fluxmi_moe_route_sort(choosed_experts.data_ptr<int32_t>(), ntokens, topk, static_cast<int32_t>(nexperts),
                                     splits.data_ptr<int32_t>(), nullptr, scatter.data_ptr<int32_t>(),
                                     gather.data_ptr<int32_t>(), topk_index.data_ptr<int32_t>(), ws.data_ptr(),
                                     ws_bytes, current_stream()),
               "fluxmi_moe_route_sort");
  return {splits, scatter, gather, topk_index};
}

// ------------------------------------------------------------------------------------------------
// Block-scaled fp8 GEMM
// ------------------------------------------------------------------------------------------------
BlockScaleGemm::BlockScaleGemm(at::ScalarType input_dtype, at::ScalarType weight_dtype, at::ScalarType output_dtype,
                               int32_t /*num_streams*/)
    : input_dtype_(input_dtype), weight_dtype_(weight_dtype), output_dtype_(output_dtype) {
  TORCH_CHECK(is_fp8(input_dtype) && is_fp8(weight_dtype), "BlockScaleGemm: input and weight must be float8_e4m3fn");
  TORCH_CHECK(output_dtype == at::kBFloat16 || output_dtype == at::kFloat,
              "BlockScaleGemm: output dtype must be bfloat16 or float32, got ", output_dtype);
}

static torch::Tensor blockscale_run(const torch::Tensor &input, const torch::Tensor &weight3, const torch::Tensor &splits_cpu,
                                    std::optional<torch::Tensor> output, const torch::Tensor &input_scale,
                                    int32_t a_layout, const torch::Tensor &weight_scale, int32_t b_layout,
                                    at::ScalarType out_dtype) {
  const int64_t m = input.size(0), k = input.size(1), e = weight3.size(0), n = weight3.size(1);
  TORCH_CHECK(weight3.size(2) == k, "weight 2-dim mismatch: ", weight3.size(2), " != ", k);
  TORCH_CHECK(k % kBlock == 0, "K must be a multiple of 128, got ", k);
  FLUX_AMD_CHECK_INPUT(input_scale, at::kFloat);
  FLUX_AMD_CHECK_INPUT(weight_scale, at::kFloat);
  const int64_t kb = k / kBlock, nb = (n + kBlock - 1) / kBlock, mb = (m + kBlock - 1) / kBlock;
  // The layout is taken from the rank, so the shape has to be exactly that layout's: a tensor of the right size in
  // another arrangement (a [E, K/128, N/128] weight scale, a natural [M, K/128] input scale) would be read wrongly
  // without any error.
  if (b_layout == FLUXMI_BSCALE_COL_N_K) {
    TORCH_CHECK(weight_scale.dim() == 4 && weight_scale.size(0) == e && weight_scale.size(1) == nb && weight_scale.size(2) == kb &&
                    weight_scale.size(3) == kBlock,
                "per-column weight_scale must be [ceil(N/128), K/128, 128] = [", nb, ", ", kb, ", ", kBlock, "]; got ",
                weight_scale.sizes());
  } else if (b_layout == FLUXMI_BSCALE_N_K) {
    TORCH_CHECK(weight_scale.dim() == 3 && weight_scale.size(0) == e && weight_scale.size(1) == nb && weight_scale.size(2) == kb,
                "weight_scale must be a 3-D tensor [E, ceil(N/128), K/128] = [", e, ", ", nb, ", ", kb,
                "] (as Quantization returns it) or the reference's flat 1-D [E * K/128 * N/128]; got ", weight_scale.sizes());
  } else {
    TORCH_CHECK(weight_scale.dim() == 1 && weight_scale.numel() == e * nb * kb,
                "weight_scale must be a 3-D tensor [E, ceil(N/128), K/128] or the reference's flat 1-D tensor of ",
                e * nb * kb, " entries ([E, K/128, N/128]); got ", weight_scale.sizes());
  }
  if (a_layout == FLUXMI_ASCALE_BLOCK128) {
    TORCH_CHECK(input_scale.dim() == 3 && input_scale.size(0) == mb && input_scale.size(1) == kb && input_scale.size(2) == kBlock,
                "input_scale must be a 3-D tensor [ceil(M/128), K/128, 128] = [", mb, ", ", kb, ", ", kBlock,
                "] (as Quantization returns it) or the reference's flat 1-D tensor (per expert [K/128, M_e]); got ",
                input_scale.sizes());
  } else {
    TORCH_CHECK(input_scale.dim() == 1 && input_scale.numel() == m * kb,
                "input_scale must be a 3-D tensor [ceil(M/128), K/128, 128] or the reference's flat 1-D tensor of ", m * kb,
                " entries (per expert [K/128, M_e], experts back to back); got ", input_scale.sizes());
  }
  torch::Tensor out;
  if (output.has_value()) {
    out = *output;
    FLUX_AMD_CHECK_INPUT(out, out_dtype);
    FLUX_AMD_CHECK_2D(out, m, n);
  } else {
    out = torch::empty({m, n}, input.options().dtype(out_dtype));
  }
  if (m == 0) return out;
  torch::Tensor splits_dev = splits_cpu.to(at::kInt).to(input.device(), /*non_blocking=*/true);
  fluxmi_grouped_gemm_args args{};
  args.dtype = FLUXMI_FP8_E4M3;
  args.nexperts = static_cast<int32_t>(e);
  args.max_rows = static_cast<int32_t>(m);
  args.n = static_cast<int32_t>(n);
  args.k = static_cast<int32_t>(k);
  args.a_rows = static_cast<int32_t>(m);
  args.a = input.data_ptr();
  args.b = weight3.data_ptr();
  args.d = out.data_ptr();
  args.splits = splits_dev.data_ptr<int32_t>();
  args.scalar_scale = 1.0f;
  args.d_fp32 = out_dtype == at::kFloat ? 1 : 0;
  check_status(fluxmi_grouped_gemm_blockscale(&args, input_scale.data_ptr<float>(), a_layout,
                                              weight_scale.data_ptr<float>(), b_layout, current_stream()),
               "fluxmi_grouped_gemm_blockscale");
  return out;
}

torch::Tensor BlockScaleGemm::forward(torch::Tensor input, torch::Tensor weight, std::optional<torch::Tensor> bias,
                                      std::optional<torch::Tensor> output, std::optional<torch::Tensor> input_scale,
                                      std::optional<torch::Tensor> weight_scale) {
  TORCH_CHECK(!bias.has_value(), "BlockScaleGemm: bias is not supported");  // as in the reference
  TORCH_CHECK(input_scale.has_value() && weight_scale.has_value(), "BlockScaleGemm: input_scale and weight_scale are required");
  FLUX_AMD_CHECK_INPUT(input, input_dtype_);
  FLUX_AMD_CHECK_INPUT(weight, weight_dtype_);
  FLUX_AMD_CHECK_NDIM(input, 2);
  FLUX_AMD_CHECK_NDIM(weight, 2);
  torch::Tensor splits = torch::full({1}, input.size(0), at::TensorOptions().dtype(at::kInt));
  TORCH_CHECK(weight_scale->dim() == 2, "weight_scale must be [ceil(N/128), K/128], got ", weight_scale->sizes());
  return blockscale_run(input, weight.unsqueeze(0), splits, output, *input_scale, FLUXMI_ASCALE_BLOCK128,
                        weight_scale->unsqueeze(0), FLUXMI_BSCALE_N_K, output_dtype_);
}

torch::Tensor BlockScaleGemm::forward_grouped(torch::Tensor input, torch::Tensor input_splits, torch::Tensor weight,
                                              std::optional<torch::Tensor> bias, std::optional<torch::Tensor> output,
                                              torch::Tensor input_scale, torch::Tensor weight_scale) {
  TORCH_CHECK(!bias.has_value(), "BlockScaleGemm: bias is not supported");
  FLUX_AMD_CHECK_INPUT(input, input_dtype_);
  FLUX_AMD_CHECK_INPUT(weight, weight_dtype_);
  FLUX_AMD_CHECK_NDIM(input, 2);
  FLUX_AMD_CHECK_NDIM(weight, 3);
  FLUX_AMD_CHECK_NDIM(input_splits, 1);
  TORCH_CHECK(!input_splits.is_cuda(), "input splits is not on cpu");
  TORCH_CHECK(input_splits.size(0) == weight.size(0), "splits 0-dim mismatch: ", input_splits.size(0), " != ",
              weight.size(0));
  TORCH_CHECK(input_splits.sum().item<int64_t>() <= input.size(0), "input_splits sum exceeds the rows of input");
  TORCH_CHECK(input_scale.dim() == 3 || input_scale.dim() == 1, "input_scale must be 3-D [ceil(M/128), K/128, 128] or the "
              "reference's flat 1-D layout (per expert [K/128, M_e]); got ", input_scale.sizes());
  TORCH_CHECK(weight_scale.dim() == 3 || weight_scale.dim() == 1, "weight_scale must be 3-D [E, ceil(N/128), K/128] or the "
              "reference's flat 1-D layout ([E, K/128, N/128]); got ", weight_scale.sizes());
  const int32_t a_layout = input_scale.dim() == 3 ? FLUXMI_ASCALE_BLOCK128 : FLUXMI_ASCALE_EXPERT_K_M;
  const int32_t b_layout = weight_scale.dim() == 3 ? FLUXMI_BSCALE_N_K : FLUXMI_BSCALE_K_N;
  return blockscale_run(input, weight, input_splits, output, input_scale, a_layout, weight_scale, b_layout, output_dtype_);
}

// The reference runs this form as one GEMM per expert spread over its streams (blockscale_gemm.cc:376-486); here it
// is the same single launch as forward_grouped.  input_scale is [M, K/128] with any strides (the reference's callers
// pass the transposed view of a [K/128, M] tensor, :440-447), weight_scale [E, N/128, K/128].
torch::Tensor BlockScaleGemm::forward_multistream(torch::Tensor input, torch::Tensor input_splits, torch::Tensor weight,
                                                  std::optional<torch::Tensor> bias, std::optional<torch::Tensor> output,
                                                  std::optional<torch::Tensor> input_scale,
                                                  std::optional<torch::Tensor> weight_scale) {
  TORCH_CHECK(!bias.has_value(), "BlockScaleGemm: bias is not supported");
  TORCH_CHECK(input_scale.has_value(), "cur_input_scale is required but missing!");
  TORCH_CHECK(weight_scale.has_value(), "BlockScaleGemm: weight_scale is required");
  FLUX_AMD_CHECK_INPUT(input, input_dtype_);
  FLUX_AMD_CHECK_INPUT(weight, weight_dtype_);
  FLUX_AMD_CHECK_NDIM(input, 2);
  FLUX_AMD_CHECK_NDIM(weight, 3);
  FLUX_AMD_CHECK_NDIM(input_splits, 1);
  FLUX_AMD_CHECK_NDIM((*input_scale), 2);
  FLUX_AMD_CHECK_NDIM((*weight_scale), 3);
  TORCH_CHECK(!input_splits.is_cuda(), "input splits is not on cpu");
  TORCH_CHECK(input_splits.size(0) == weight.size(0), "splits 0-dim mismatch: ", input_splits.size(0), " != ",
              weight.size(0));
  TORCH_CHECK(input_splits.sum().item<int64_t>() <= input.size(0), "input_splits sum exceeds the rows of input");
  const int64_t m = input.size(0), kb = input.size(1) / kBlock;
  TORCH_CHECK(input_scale->is_cuda() && input_scale->scalar_type() == at::kFloat && input_scale->size(0) == m &&
                  input_scale->size(1) == kb,
              "input_scale must be a float32 device tensor of shape [", m, ", ", kb, "]");
  // [M, K/128] -> [ceil(M/128), K/128, 128], the layout the kernel reads rows of scales from.
  const int64_t mb = (m + kBlock - 1) / kBlock;
  torch::Tensor padded = torch::zeros({mb * kBlock, kb}, input_scale->options());
  padded.narrow(0, 0, m).copy_(*input_scale);
  torch::Tensor blocked = padded.view({mb, kBlock, kb}).permute({0, 2, 1}).contiguous();
  return blockscale_run(input, weight, input_splits, output, blocked, FLUXMI_ASCALE_BLOCK128, weight_scale->contiguous(),
                        FLUXMI_BSCALE_N_K, output_dtype_);
}

// The reference's second implementation of forward (blockscale_gemm.cc:954-973); one kernel serves both here.  With
// is_groupwise_b the weight carries one scale per column and 128 of K, [ceil(N/128), K/128, 128] (the
// ScaleNsPerTile == BLOCK_N case of test/python/gemm_only/test_blockwise_scale_gemm_only.py:209,237-240): that form
// runs on the generic kernel (a checking path, as `reference` is in the reference).
torch::Tensor BlockScaleGemm::reference(torch::Tensor input, torch::Tensor weight, std::optional<torch::Tensor> bias,
                                        std::optional<torch::Tensor> output, std::optional<torch::Tensor> input_scale,
                                        std::optional<torch::Tensor> weight_scale, bool is_groupwise_b) {
  if (!is_groupwise_b)
    return forward(std::move(input), std::move(weight), std::move(bias), std::move(output), std::move(input_scale),
                   std::move(weight_scale));
  TORCH_CHECK(!bias.has_value(), "BlockScaleGemm: bias is not supported");
  TORCH_CHECK(input_scale.has_value() && weight_scale.has_value(), "BlockScaleGemm: input_scale and weight_scale are required");
  FLUX_AMD_CHECK_INPUT(input, input_dtype_);
  FLUX_AMD_CHECK_INPUT(weight, weight_dtype_);
  FLUX_AMD_CHECK_NDIM(input, 2);
  FLUX_AMD_CHECK_NDIM(weight, 2);
  TORCH_CHECK(weight_scale->dim() == 3, "per-column weight_scale must be [ceil(N/128), K/128, 128], got ", weight_scale->sizes());
  torch::Tensor splits = torch::full({1}, input.size(0), at::TensorOptions().dtype(at::kInt));
  return blockscale_run(input, weight.unsqueeze(0), splits, output, *input_scale, FLUXMI_ASCALE_BLOCK128,
                        weight_scale->unsqueeze(0), FLUXMI_BSCALE_COL_N_K, output_dtype_);
}

// The reference times every registered kernel configuration and runs the best (blockscale_gemm.cc:975-1023); there is
// one configuration here, so this is forward.
torch::Tensor BlockScaleGemm::profiling(torch::Tensor input, torch::Tensor weight, std::optional<torch::Tensor> bias,
                                        std::optional<torch::Tensor> output, std::optional<torch::Tensor> input_scale,
                                        std::optional<torch::Tensor> weight_scale, std::shared_ptr<ProfilingContext>) {
  return forward(std::move(input), std::move(weight), std::move(bias), std::move(output), std::move(input_scale),
                 std::move(weight_scale));
}

torch::Tensor calc_scatter_index(torch::Tensor choosed_experts, torch::Tensor splits) {
  FLUX_AMD_CHECK_INPUT(choosed_experts, at::kInt);
  FLUX_AMD_CHECK_INPUT(splits, at::kInt);
  torch::Tensor flat = choosed_experts.dim() == 2 ? choosed_experts : choosed_experts.reshape({-1, 1});
  // The reference's kernel orders pairs inside an expert by atomics (src/cuda/moe_utils.cu:48-61); this
  // one returns the stable order, which is one of the orders that kernel may produce.
  auto r = moe_route_sort(flat, splits.numel());
  return std::get<1>(r).reshape(choosed_experts.sizes());
}

torch::Tensor topk_weighted_gather_reduce(std::vector<torch::Tensor> inputs, torch::Tensor routing_idx, int64_t topk,
                                          std::optional<torch::Tensor> row_weight, double scale) {
  TORCH_CHECK(!inputs.empty(), "inputs must not be empty");
  const at::ScalarType st = inputs[0].scalar_type();
  TORCH_CHECK(st == at::kBFloat16 || st == at::kFloat || st == at::kHalf, "inputs must be bfloat16, float16 or float32");
  const int64_t m = inputs[0].size(0), n = inputs[0].size(1);
  TORCH_CHECK(topk >= 1 && m % topk == 0, "rows ", m, " not a multiple of topk ", topk);
  FLUX_AMD_CHECK_INPUT(routing_idx, at::kInt);
  TORCH_CHECK(routing_idx.numel() == m, "routing index must have one entry per input row");
  std::vector<const void *> ptrs;
  for (auto &t : inputs) {
    FLUX_AMD_CHECK_INPUT(t, st);
    FLUX_AMD_CHECK_2D(t, m, n);
    ptrs.push_back(t.data_ptr());
  }
  const float *w = nullptr;
  if (row_weight.has_value()) {
    FLUX_AMD_CHECK_INPUT(*row_weight, at::kFloat);
    TORCH_CHECK(row_weight->numel() == m, "row_weight must be [M]");
    w = row_weight->data_ptr<float>();
  }
  torch::Tensor out = torch::empty({m / topk, n}, inputs[0].options().dtype(st == at::kHalf ? at::kHalf : at::kBFloat16));
  check_status(fluxmi_topk_gather_reduce(ptrs.data(), static_cast<int32_t>(ptrs.size()), st == at::kFloat ? 1 : (st == at::kHalf ? 2 : 0),
                                         routing_idx.data_ptr<int32_t>(), w, static_cast<float>(scale),
                                         static_cast<int32_t>(m / topk), static_cast<int32_t>(topk),
                                         static_cast<int32_t>(n), out.data_ptr(), current_stream()),
               "fluxmi_topk_gather_reduce");
  return out;
}

torch::Tensor topk_scatter_reduce(std::vector<torch::Tensor> inputs, torch::Tensor scatter_idx, int64_t topk) {
  return topk_weighted_gather_reduce(inputs, scatter_idx.reshape({-1}), topk, std::nullopt, 1.0);
}

bool bitwise_check(torch::Tensor a, torch::Tensor b) {
  if (a.sizes() != b.sizes() || a.scalar_type() != b.scalar_type()) return false;
  auto av = a.contiguous().view(at::kByte).reshape({-1});
  auto bv = b.contiguous().view(at::kByte).reshape({-1});
  return torch::equal(av, bv);
}

}  // namespace flux_amd
