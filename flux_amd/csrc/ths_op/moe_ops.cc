// The reference's MoE operator classes rebuilt over the C-ABI (include/fluxmi.h):
//   GemmGroupedV3AGScatter  src/moe_ag_scatter/ths_op/gemm_grouped_v3_ag_scatter.{h,cc}
//   GemmGroupedV3GatherRS   src/moe_gather_rs/ths_op/gemm_grouped_v3_gather_rs.{h,cc}
//   GemmGroupedV3           src/comm_none/ths_op/gemm_grouped_v3.cc:43-171
// Same constructor and method signatures, same argument checks; every launch goes to the current HIP
// stream and nothing synchronises the host (the reference's layer0 blocks once to read the splits back,
// gemm_grouped_v3_ag_scatter.cc:323-331 — here the tile schedule is built on the device).
#include <algorithm>
#include <cstdlib>

#include <hip/hip_runtime_api.h>

#include "ths_ops.h"

namespace flux_amd {

namespace {
// Schedule forced on every launch of this thread while a profiler tries it.
thread_local const GemmLaunchTuning *t_tuning_override = nullptr;
// Form of layer1's reduction forced on this thread while a profiler tries it: 0 none, 1 fused, 2 two-pass.
thread_local int t_reduce_override = 0;

struct ScopedReduceOverride {
  explicit ScopedReduceOverride(int form) { t_reduce_override = form; }
  ~ScopedReduceOverride() { t_reduce_override = 0; }
};

struct ScopedTuningOverride {
  explicit ScopedTuningOverride(const GemmLaunchTuning *t) { t_tuning_override = t; }
  ~ScopedTuningOverride() { t_tuning_override = nullptr; }
};

GemmShapeKey shape_key(const fluxmi_grouped_gemm_args &args, int32_t ngroups) {
  GemmShapeKey key;
  key.dtype = args.dtype;
  key.nexperts = args.nexperts;
  key.n = args.n;
  key.k = args.k;
  key.max_rows = args.max_rows;
  key.ngroups = ngroups;
  return key;
}

#define FLUX_AMD_HIP_CHECK(expr)                                                                          \
  do {                                                                                                    \
    const hipError_t err_ = (expr);                                                                       \
    if (err_ != hipSuccess) throw std::runtime_error(std::string(#expr " failed: ") + hipGetErrorString(err_)); \
  } while (0)

// Times `run` (one whole forward) under every candidate schedule on the current stream, 5 warm-up and 10
// timed calls each like the reference's profiling loops (gemm_grouped_v3_ag_scatter.cc:540-590), records
// them in `ctx` and registers the fastest for `key`.
// Mean time in ms of one call of `run` on the current stream: 5 warm-up and 10 timed calls.
template <class F>
float time_calls(F &&run) {
  constexpr int kWarmIters = 5, kIters = 10;
  hipStream_t stream = static_cast<hipStream_t>(current_stream());
  hipEvent_t e0, e1;
  FLUX_AMD_HIP_CHECK(hipEventCreate(&e0));
  FLUX_AMD_HIP_CHECK(hipEventCreate(&e1));
  float ms = 0.f;
  try {
    for (int i = 0; i < kWarmIters; ++i) run();
    FLUX_AMD_HIP_CHECK(hipEventRecord(e0, stream));
    for (int i = 0; i < kIters; ++i) run();
    FLUX_AMD_HIP_CHECK(hipEventRecord(e1, stream));
    FLUX_AMD_HIP_CHECK(hipEventSynchronize(e1));
    FLUX_AMD_HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
  } catch (...) {
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    throw;
  }
  FLUX_AMD_HIP_CHECK(hipEventDestroy(e0));
  FLUX_AMD_HIP_CHECK(hipEventDestroy(e1));
  return ms / kIters;
}

template <class F>
void profile_schedules(const GemmShapeKey &key, ProfilingContext *ctx, F &&run) {
  for (const GemmLaunchTuning &cand : gemm_tuning_candidates()) {
    ScopedTuningOverride scope(&cand);
    ctx->add(key, cand, time_calls(run));
  }
  TuningTable::instance().add(key, ctx->record_best(key));
}
}  // namespace

void apply_launch_tuning(fluxmi_grouped_gemm_args &args, int32_t ngroups, int64_t sm_margin) {
  TORCH_CHECK(sm_margin >= 0 && sm_margin < (1 << 20), "sm_margin must be non-negative, got ", sm_margin);
  args.cu_margin = static_cast<int32_t>(sm_margin);
  if (t_tuning_override != nullptr) {
    args.raster_rows = t_tuning_override->raster_rows;
    args.sched_flags = t_tuning_override->sched_flags;
  } else if (auto t = TuningTable::instance().find(shape_key(args, ngroups))) {
    args.raster_rows = t->raster_rows;
    args.sched_flags = t->sched_flags;
  }
}

void run_grouped_gemm(const torch::Tensor &a, const torch::Tensor &b, const torch::Tensor &splits_dev,
                      torch::Tensor &d, const int32_t *gather_a, int64_t max_rows, const float *alpha,
                      const float *row_scale, const float *col_scale, const float *scalar_dev,
                      int64_t sm_margin) {
  fluxmi_grouped_gemm_args args{};
  args.dtype = to_fluxmi_dtype(a.scalar_type());
  args.nexperts = static_cast<int32_t>(b.size(0));
  args.max_rows = static_cast<int32_t>(max_rows);
  args.n = static_cast<int32_t>(b.size(1));
  args.k = static_cast<int32_t>(b.size(2));
  args.a_rows = static_cast<int32_t>(a.size(0));
  args.a = a.data_ptr();
  args.b = b.data_ptr();
  args.d = d.data_ptr();
  args.splits = splits_dev.data_ptr<int32_t>();
  args.gather_a = gather_a;
  args.scatter_d = nullptr;
  args.alpha = alpha;
  args.row_scale = row_scale;
  args.col_scale = col_scale;
  args.scalar_scale = 1.0f;
  args.d_fp32 = d.scalar_type() == at::ScalarType::Float ? 1 : 0;
  args.scalar_scale_dev = scalar_dev;
  apply_launch_tuning(args, 1, sm_margin);
  check_status(fluxmi_grouped_gemm(&args, nullptr, 0, current_stream()), "fluxmi_grouped_gemm");
}

// ------------------------------------------------------------------------------------------------
// Layer0: gather + grouped GEMM
// ------------------------------------------------------------------------------------------------
GemmGroupedV3AGScatter::GemmGroupedV3AGScatter(DistEnvTPWithEP tp_env, MoeArguments moe_args)
    : tp_env_(tp_env), moe_args_(moe_args) {
  TORCH_CHECK(moe_args.max_ntokens > 0 && moe_args.hidden > 0 && moe_args.ffn_hidden > 0 &&
                  moe_args.nexperts > 0 && moe_args.topk > 0,
              "MoeArguments sizes must be positive");
  to_fluxmi_dtype(moe_args.input_dtype);
  TORCH_CHECK(moe_args.output_dtype == moe_output_dtype(moe_args.input_dtype),
              "output dtype must be ", moe_output_dtype(moe_args.input_dtype), " for ", moe_args.input_dtype,
              " inputs (fp16 gives fp16; bf16 and fp8 give bf16), got ", moe_args.output_dtype);
  // Persistent scratch sized from the constructor arguments, like the reference's input_buffer
  // (gemm_grouped_v3_ag_scatter.cc:86-101): the inverse permutation of scatter_index.
  gather_index_ = torch::empty({static_cast<int64_t>(moe_args.max_ntokens) * moe_args.topk},
                               at::TensorOptions().dtype(at::kInt).device(at::kCUDA));
}

void GemmGroupedV3AGScatter::clear_buffers() {}  // no flags or symmetric buffers exist at world size 1

std::vector<torch::Tensor> GemmGroupedV3AGScatter::forward_impl(
    torch::Tensor inputs_shard, std::vector<torch::Tensor> weights, torch::Tensor splits_gpu,
    torch::Tensor scatter_index, std::optional<std::vector<torch::Tensor>> output_scale,
    std::optional<std::vector<torch::Tensor>> outputs_buf, std::optional<torch::Tensor> allgather_output,
    bool /*fast_accum*/, int64_t sm_margin) {
  FLUX_AMD_CHECK_INPUT(inputs_shard, moe_args_.input_dtype);
  FLUX_AMD_CHECK_NDIM(inputs_shard, 2);
  const int64_t ntokens = inputs_shard.size(0);  // world size 1: the shard is the whole batch
  FLUX_AMD_CHECK_2D(inputs_shard, ntokens, moe_args_.hidden);
  TORCH_CHECK(ntokens <= moe_args_.max_ntokens, "ntokens ", ntokens, " exceeds max_ntokens ",
              moe_args_.max_ntokens);
  TORCH_CHECK(!weights.empty(), "weights must not be empty");
  const size_t groups = weights.size();
  for (size_t i = 0; i < groups; ++i) {
    FLUX_AMD_CHECK_INPUT(weights[i], moe_args_.input_dtype);
    FLUX_AMD_CHECK_3D(weights[i], moe_args_.nexperts, moe_args_.ffn_hidden, moe_args_.hidden);
  }
  FLUX_AMD_CHECK_INPUT(splits_gpu, at::kInt);
  FLUX_AMD_CHECK_NDIM(splits_gpu, 1);
  TORCH_CHECK(splits_gpu.size(0) >= moe_args_.nexperts, "splits_gpu has ", splits_gpu.size(0),
              " entries, expected at least ", moe_args_.nexperts);
  FLUX_AMD_CHECK_INPUT(scatter_index, at::kInt);
  FLUX_AMD_CHECK_2D(scatter_index, ntokens, moe_args_.topk);
  if (output_scale.has_value()) {
    TORCH_CHECK(output_scale->size() == groups, "output_scale needs one tensor per weight group");
    for (size_t i = 0; i < groups; ++i) {
      FLUX_AMD_CHECK_INPUT(output_scale->at(i), at::kFloat);
      TORCH_CHECK(output_scale->at(i).dim() == 1 && output_scale->at(i).size(0) == moe_args_.nexperts,
                  "output_scale must be [nexperts]");
    }
  }
  const int64_t nrows = ntokens * moe_args_.topk;  // total_nrows_ep at ep size 1
  std::vector<torch::Tensor> outputs;
  if (outputs_buf.has_value()) {
    TORCH_CHECK(outputs_buf->size() == groups, "outputs_buf needs one tensor per weight group");
    for (size_t i = 0; i < groups; ++i) {
      FLUX_AMD_CHECK_INPUT(outputs_buf->at(i), moe_args_.output_dtype);
      TORCH_CHECK(outputs_buf->at(i).dim() == 2 && outputs_buf->at(i).size(0) >= nrows &&
                      outputs_buf->at(i).size(1) == moe_args_.ffn_hidden,
                  "outputs_buf[", i, "] shape ", outputs_buf->at(i).sizes(), " too small for [", nrows, ", ",
                  moe_args_.ffn_hidden, "]");
      outputs.push_back(outputs_buf->at(i));
    }
  } else {
    for (size_t i = 0; i < groups; ++i)
      outputs.push_back(torch::empty({nrows, moe_args_.ffn_hidden},
                                     inputs_shard.options().dtype(moe_args_.output_dtype)));
  }
  if (nrows > 0) {
    // K2 of the reference (calc_gather_index_impl, sort_util.cu:121-160); the (rank, expert) bucket
    // sort that follows it there is the identity at world size 1.
    check_status(fluxmi_moe_gather_index(scatter_index.data_ptr<int32_t>(), static_cast<int32_t>(nrows),
                                         moe_args_.topk, gather_index_.data_ptr<int32_t>(), nullptr,
                                         current_stream()),
                 "fluxmi_moe_gather_index");
    // All weight groups (gate and up projections, say) run as one launch over one tile schedule: the
    // gathered A tiles an XCD's L2 holds serve every group, and the launch has one tail instead of one per
    // group (the reference shares the gathered A the same way, gemm_grouped_v3_ag_scatter.cc:375-395).
    constexpr size_t kMaxGroupsPerLaunch = 4;
    for (size_t g0 = 0; g0 < groups; g0 += kMaxGroupsPerLaunch) {
      const size_t ng = std::min(kMaxGroupsPerLaunch, groups - g0);
      const void *b[kMaxGroupsPerLaunch];
      void *d[kMaxGroupsPerLaunch];
      const float *alpha[kMaxGroupsPerLaunch];
      for (size_t i = 0; i < ng; ++i) {
        b[i] = weights[g0 + i].data_ptr();
        d[i] = outputs[g0 + i].data_ptr();
        alpha[i] = output_scale.has_value() ? output_scale->at(g0 + i).data_ptr<float>() : nullptr;
      }
      fluxmi_grouped_gemm_args args{};
      args.dtype = to_fluxmi_dtype(inputs_shard.scalar_type());
      args.nexperts = static_cast<int32_t>(moe_args_.nexperts);
      args.max_rows = static_cast<int32_t>(nrows);
      args.n = static_cast<int32_t>(moe_args_.ffn_hidden);
      args.k = static_cast<int32_t>(moe_args_.hidden);
      args.a_rows = static_cast<int32_t>(ntokens);
      args.a = inputs_shard.data_ptr();
      args.splits = splits_gpu.data_ptr<int32_t>();
      args.gather_a = gather_index_.data_ptr<int32_t>();
      args.scalar_scale = 1.0f;
      apply_launch_tuning(args, static_cast<int32_t>(ng), sm_margin);
      check_status(fluxmi_grouped_gemm_multi(&args, static_cast<int32_t>(ng), b, d, alpha, nullptr, 0,
                                             current_stream()),
                   "fluxmi_grouped_gemm_multi");
    }
  }
  if (allgather_output.has_value()) {  // gemm_grouped_v3_ag_scatter.cc:440-445
    TORCH_CHECK(allgather_output->sizes() == inputs_shard.sizes(), "allgather_output shape mismatch");
    allgather_output->copy_(inputs_shard);
  }
  return outputs;
}

torch::Tensor GemmGroupedV3AGScatter::forward(torch::Tensor inputs_shard, torch::Tensor weights,
                                              torch::Tensor splits_gpu, torch::Tensor scatter_index,
                                              std::optional<torch::Tensor> output_scale,
                                              std::optional<torch::Tensor> outputs_buf,
                                              std::optional<torch::Tensor> allgather_output,
                                              bool fast_accum, int64_t sm_margin) {
  std::optional<std::vector<torch::Tensor>> scales, bufs;
  if (output_scale.has_value()) scales = std::vector<torch::Tensor>{*output_scale};
  if (outputs_buf.has_value()) bufs = std::vector<torch::Tensor>{*outputs_buf};
  return forward_impl(inputs_shard, {weights}, splits_gpu, scatter_index, scales, bufs, allgather_output,
                      fast_accum, sm_margin)[0];
}

std::vector<torch::Tensor> GemmGroupedV3AGScatter::forward_multiple_weights(
    torch::Tensor inputs_shard, std::vector<torch::Tensor> weights, torch::Tensor splits_gpu,
    torch::Tensor scatter_index, std::optional<std::vector<torch::Tensor>> output_scale,
    std::optional<std::vector<torch::Tensor>> outputs_buf, std::optional<torch::Tensor> allgather_output,
    bool fast_accum, int64_t sm_margin) {
  return forward_impl(inputs_shard, weights, splits_gpu, scatter_index, output_scale, outputs_buf,
                      allgather_output, fast_accum, sm_margin);
}

torch::Tensor GemmGroupedV3AGScatter::profiling(torch::Tensor inputs_shard, torch::Tensor weights,
                                                torch::Tensor splits_gpu, torch::Tensor scatter_index,
                                                std::optional<torch::Tensor> output_scale,
                                                std::optional<torch::Tensor> outputs_buf,
                                                std::optional<torch::Tensor> allgather_output, bool fast_accum,
                                                int64_t sm_margin, std::shared_ptr<ProfilingContext> prof_ctx) {
  ProfilingContext tmp_ctx("__tmp__");
  ProfilingContext *ctx = prof_ctx ? prof_ctx.get() : &tmp_ctx;
  auto run = [&]() {
    return forward(inputs_shard, weights, splits_gpu, scatter_index, output_scale, outputs_buf, allgather_output,
                   fast_accum, sm_margin);
  };
  run();  // argument checks before anything is timed
  GemmShapeKey key;
  key.dtype = to_fluxmi_dtype(moe_args_.input_dtype);
  key.nexperts = moe_args_.nexperts;
  key.n = moe_args_.ffn_hidden;
  key.k = moe_args_.hidden;
  key.max_rows = static_cast<int32_t>(inputs_shard.size(0) * moe_args_.topk);
  key.ngroups = 1;
  if (key.max_rows > 0) profile_schedules(key, ctx, run);
  return run();  // with the schedule just registered
}

// ------------------------------------------------------------------------------------------------
// Layer1: grouped GEMM + top-k gather-reduce
// ------------------------------------------------------------------------------------------------
GemmGroupedV3GatherRS::GemmGroupedV3GatherRS(int64_t total_num_experts, int64_t max_m, int64_t n_dim,
                                             int64_t topk, int64_t rank, int64_t world_size,
                                             int64_t tp_world_size, int64_t ep_world_size,
                                             int64_t max_input_groups, bool ep_in_dp)
    : num_experts_(total_num_experts), max_m_(max_m), n_dim_(n_dim), topk_(topk),
      max_input_groups_(max_input_groups) {
  TORCH_CHECK(rank == 0 && world_size == 1 && tp_world_size == 1 && ep_world_size == 1 && !ep_in_dp,
              "GemmGroupedV3GatherRS: this build runs on one GPU only (rank=0, world_size=1, "
              "tp_world_size=1, ep_world_size=1, ep_in_dp=False), got rank=", rank, " world_size=",
              world_size, " tp=", tp_world_size, " ep=", ep_world_size);
  TORCH_CHECK(total_num_experts > 0 && max_m > 0 && n_dim > 0 && topk > 0, "sizes must be positive");
  TORCH_CHECK(max_input_groups >= 1 && max_input_groups <= 4, "max_input_groups must be in [1, 4]");
  const char *env = std::getenv("FLUX_AMD_INTER_DTYPE");
  inter_fp32_ = !(env != nullptr && std::string(env) == "bf16");
  // Where the top-k reduction happens: in the GEMM's epilogue (atomic adds into an fp32 [T, N] buffer, the
  // reference's fused form) or in a gather-reduce kernel after the GEMM (deterministic for every top-k).
  const char *red = std::getenv("FLUX_AMD_LAYER1_REDUCE");
  if (red != nullptr && std::string(red) == "fused") fused_mode_ = 1;
  else if (red != nullptr && std::string(red) == "twopass") fused_mode_ = 2;
  else TORCH_CHECK(red == nullptr || std::string(red).empty(), "FLUX_AMD_LAYER1_REDUCE must be 'fused' or 'twopass', got ", red);
}

void GemmGroupedV3GatherRS::lazy_init(const torch::Tensor &like) {
  if (!inter_.empty()) return;
  // inter_D of the reference (gemm_grouped_v3_gather_rs.cc:165-232) is bf16; the default here is fp32 so
  // that the layer has a single rounding.  FLUX_AMD_INTER_DTYPE=bf16 restores the reference's data flow.
  // Zero-filled once, as the reference does (init_buffer: torch::zeros): rows the GEMM never writes
  // (sum(splits) < M) then read as zeros in the reduce instead of stale memory.
  auto opts = like.options().dtype(inter_fp32_ ? at::kFloat : moe_output_dtype(like.scalar_type()));
  for (int64_t g = 0; g < max_input_groups_; ++g) inter_.push_back(torch::zeros({max_m_, n_dim_}, opts));
  splits_dev_ = torch::empty({num_experts_}, like.options().dtype(at::kInt));
  token_of_row_ = torch::empty({max_m_}, like.options().dtype(at::kInt));
}

torch::Tensor GemmGroupedV3GatherRS::forward_impl(
    std::vector<torch::Tensor> inputs, std::vector<torch::Tensor> weights, torch::Tensor splits_cpu,
    torch::Tensor routing_idx, std::optional<std::vector<torch::Tensor>> input_scale,
    std::optional<std::vector<torch::Tensor>> weight_scale,
    std::optional<std::vector<torch::Tensor>> output_vec_scale, bool with_stream_sync, int64_t sm_margin) {
  TORCH_CHECK(!inputs.empty() && inputs.size() == weights.size(), "inputs / weights group count mismatch");
  TORCH_CHECK(static_cast<int64_t>(inputs.size()) <= max_input_groups_, "more input groups than max_input_groups");
  const at::ScalarType st = weights[0].scalar_type();
  to_fluxmi_dtype(st);
  const int64_t global_m = routing_idx.size(0);
  const int64_t m = inputs[0].size(0);
  const int64_t k = inputs[0].size(1);
  for (size_t i = 0; i < inputs.size(); ++i) {
    FLUX_AMD_CHECK_INPUT(weights[i], st);
    FLUX_AMD_CHECK_3D(weights[i], num_experts_, n_dim_, k);
    FLUX_AMD_CHECK_INPUT(inputs[i], st);
    FLUX_AMD_CHECK_2D(inputs[i], m, k);
  }
  TORCH_CHECK(splits_cpu.scalar_type() == at::kInt, "splits_cpu must be int32");
  TORCH_CHECK(!splits_cpu.is_cuda(), "splits_cpu must be a host tensor");
  FLUX_AMD_CHECK_NDIM(splits_cpu, 1);
  TORCH_CHECK(splits_cpu.size(0) == num_experts_, "splits 0-dim mismatch: ", splits_cpu.size(0),
              " != ", num_experts_);
  FLUX_AMD_CHECK_INPUT(routing_idx, at::kInt);
  FLUX_AMD_CHECK_NDIM(routing_idx, 1);
  TORCH_CHECK(m == global_m, "input.size(0) ", m, " != routing_idx.size(0) ", global_m);
  TORCH_CHECK(global_m % topk_ == 0, "routing_idx.size(0) must be a multiple of topk");
  TORCH_CHECK(global_m <= max_m_, "routing_idx.size(0) ", global_m, " larger than max_m ", max_m_);
  TORCH_CHECK(n_dim_ >= 8 && k >= 8, "N and K must be at least 8");
  const size_t groups = inputs.size();
  auto check_scales = [&](const std::optional<std::vector<torch::Tensor>> &s, const char *name) {
    if (!s.has_value()) return;
    TORCH_CHECK(s->size() == groups, name, " needs one tensor per input group");
    for (auto &t : *s) FLUX_AMD_CHECK_INPUT(t, at::kFloat);
  };
  check_scales(input_scale, "input_scale");
  check_scales(weight_scale, "weight_scale");
  check_scales(output_vec_scale, "output_vec_scale");

  lazy_init(inputs[0]);
  const int64_t ntokens = global_m / topk_;
  const bool f16 = st == at::ScalarType::Half;
  torch::Tensor out = torch::empty({ntokens, n_dim_}, inputs[0].options().dtype(moe_output_dtype(st)));
  if (global_m == 0) return out;
  splits_dev_.copy_(splits_cpu.contiguous(), /*non_blocking=*/true);

  // One input group and an fp32 scratch at hand: the reduction may run in the GEMM's epilogue.  It does when
  // FLUX_AMD_LAYER1_REDUCE=fused asks for it, or when profiling() found it faster for this shape (a tuning record
  // with reduce=fused); FLUX_AMD_LAYER1_REDUCE=twopass overrides the table.  Without either the two-pass form runs:
  // it is the faster one on every shape measured so far and deterministic for every top-k.
  bool want_fused = fused_mode_ == 1;
  if (fused_mode_ == 0) {
    if (t_reduce_override != 0) {
      want_fused = t_reduce_override == 1;
    } else {
      GemmShapeKey key;
      key.dtype = to_fluxmi_dtype(st);
      key.nexperts = static_cast<int32_t>(num_experts_);
      key.n = static_cast<int32_t>(n_dim_);
      key.k = static_cast<int32_t>(k);
      key.max_rows = static_cast<int32_t>(m);
      key.ngroups = 1;
      if (auto t = TuningTable::instance().find(key)) want_fused = t->reduce_fused != 0;
    }
  }
  const bool fused = want_fused && groups == 1 && inter_fp32_;
  std::vector<const void *> group_ptrs;
  for (size_t g = 0; g < groups; ++g) {
    const float *alpha = nullptr, *row = nullptr, *col = nullptr, *scalar = nullptr;
    torch::Tensor row_holder;
    if (weight_scale.has_value()) {
      const auto &ws = weight_scale->at(g);
      if (ws.numel() == num_experts_) alpha = ws.data_ptr<float>();
      else if (ws.numel() == num_experts_ * n_dim_) col = ws.data_ptr<float>();
      else TORCH_CHECK(false, "weight_scale must be [E] or [E, N]");
    }
    if (output_vec_scale.has_value()) {
      TORCH_CHECK(output_vec_scale->at(g).numel() == m, "output_vec_scale must be [M]");
      row_holder = output_vec_scale->at(g);
    }
    if (input_scale.has_value()) {
      const auto &is = input_scale->at(g);
      if (is.numel() == 1) scalar = is.data_ptr<float>();
      else if (is.numel() == m) row_holder = row_holder.defined() ? row_holder * is.reshape({m}) : is;
      else TORCH_CHECK(false, "input_scale must be [1] or [M]");
    }
    if (row_holder.defined()) row = row_holder.data_ptr<float>();
    if (fused) {
      token_of_row_.fill_(-1);  // sorted rows that no routing entry names are skipped by the epilogue
      check_status(fluxmi_moe_gather_index(routing_idx.data_ptr<int32_t>(), static_cast<int32_t>(global_m),
                                           static_cast<int32_t>(topk_), token_of_row_.data_ptr<int32_t>(), nullptr,
                                           current_stream()),
                   "fluxmi_moe_gather_index");
      fluxmi_grouped_gemm_args args{};
      args.dtype = to_fluxmi_dtype(inputs[g].scalar_type());
      args.nexperts = static_cast<int32_t>(num_experts_);
      args.max_rows = static_cast<int32_t>(m);
      args.n = static_cast<int32_t>(n_dim_);
      args.k = static_cast<int32_t>(k);
      args.a_rows = static_cast<int32_t>(m);
      args.a = inputs[g].data_ptr();
      args.b = weights[g].data_ptr();
      args.splits = splits_dev_.data_ptr<int32_t>();
      args.alpha = alpha;
      args.row_scale = row;
      args.col_scale = col;
      args.scalar_scale = 1.0f;
      args.scalar_scale_dev = scalar;
      apply_launch_tuning(args, 1, sm_margin);
      check_status(fluxmi_grouped_gemm_topk_reduce(&args, token_of_row_.data_ptr<int32_t>(), static_cast<int32_t>(ntokens),
                                                   out.data_ptr(), inter_[0].data_ptr(),
                                                   static_cast<size_t>(inter_[0].numel()) * 4, current_stream()),
                   "fluxmi_grouped_gemm_topk_reduce");
      if (with_stream_sync) c10::hip::getCurrentHIPStream().synchronize();
      return out;
    }
    run_grouped_gemm(inputs[g], weights[g], splits_dev_, inter_[g], nullptr, m, alpha, row, col, scalar, sm_margin);
    group_ptrs.push_back(inter_[g].data_ptr());
  }
  check_status(fluxmi_topk_gather_reduce(group_ptrs.data(), static_cast<int32_t>(groups), (inter_fp32_ ? 1 : 0) | (f16 ? 2 : 0),
                                         routing_idx.data_ptr<int32_t>(), nullptr, 1.0f,
                                         static_cast<int32_t>(ntokens), static_cast<int32_t>(topk_),
                                         static_cast<int32_t>(n_dim_), out.data_ptr(), current_stream()),
               "fluxmi_topk_gather_reduce");
  if (with_stream_sync) c10::hip::getCurrentHIPStream().synchronize();
  return out;
}

torch::Tensor GemmGroupedV3GatherRS::forward_gather_rs(
    torch::Tensor input, torch::Tensor weight, torch::Tensor splits_cpu, torch::Tensor routing_idx,
    std::optional<torch::Tensor> /*n_tokens_per_rank*/, std::optional<torch::Tensor> input_scale,
    std::optional<torch::Tensor> weight_scale, std::optional<torch::Tensor> output_vec_scale,
    bool /*fast_accum*/, int64_t sm_margin, bool with_stream_sync) {
  auto wrap = [](std::optional<torch::Tensor> &t) {
    std::optional<std::vector<torch::Tensor>> v;
    if (t.has_value()) v = std::vector<torch::Tensor>{*t};
    return v;
  };
  return forward_impl({input}, {weight}, splits_cpu, routing_idx, wrap(input_scale), wrap(weight_scale),
                      wrap(output_vec_scale), with_stream_sync, sm_margin);
}

torch::Tensor GemmGroupedV3GatherRS::profiling(
    torch::Tensor input, torch::Tensor weight, torch::Tensor splits_cpu, torch::Tensor routing_idx,
    std::optional<torch::Tensor> n_tokens_per_rank, std::optional<torch::Tensor> input_scale,
    std::optional<torch::Tensor> weight_scale, std::optional<torch::Tensor> output_vec_scale, bool fast_accum,
    int64_t sm_margin, bool with_stream_sync, std::shared_ptr<ProfilingContext> prof_ctx) {
  ProfilingContext tmp_ctx("__tmp__");
  ProfilingContext *ctx = prof_ctx ? prof_ctx.get() : &tmp_ctx;
  auto run = [&]() {
    return forward_gather_rs(input, weight, splits_cpu, routing_idx, n_tokens_per_rank, input_scale, weight_scale,
                             output_vec_scale, fast_accum, sm_margin, with_stream_sync);
  };
  run();  // argument checks before anything is timed
  GemmShapeKey key;
  key.dtype = to_fluxmi_dtype(weight.scalar_type());
  key.nexperts = static_cast<int32_t>(num_experts_);
  key.n = static_cast<int32_t>(n_dim_);
  key.k = static_cast<int32_t>(input.size(1));
  key.max_rows = static_cast<int32_t>(input.size(0));
  key.ngroups = 1;
  if (key.max_rows > 0) {
    {
      ScopedReduceOverride twopass(fused_mode_ == 0 ? 2 : 0);  // an earlier record must not switch forms mid-sweep
      profile_schedules(key, ctx, run);
    }
    // With the fastest schedule registered: the other form of the reduction (atomic adds in the GEMM's epilogue
    // instead of GEMM + gather-reduce kernel), when this op could run either.  Its time ranks among the two-pass
    // timings of every schedule; the fastest entry becomes the record.
    if (fused_mode_ == 0 && inter_fp32_) {
      GemmLaunchTuning best = *TuningTable::instance().find(key);
      best.reduce_fused = 1;
      float ms = 0.f;
      {
        ScopedReduceOverride fused(1);
        ms = time_calls(run);
      }
      ctx->add(key, best, ms);
      TuningTable::instance().add(key, ctx->record_best(key));
    }
  }
  return run();  // with the schedule just registered
}

torch::Tensor GemmGroupedV3GatherRS::forward_gather_rs_multiple(
    std::vector<torch::Tensor> inputs, std::vector<torch::Tensor> weights, torch::Tensor splits_cpu,
    torch::Tensor routing_idx, std::optional<torch::Tensor> /*n_tokens_per_rank*/,
    std::optional<std::vector<torch::Tensor>> input_scale,
    std::optional<std::vector<torch::Tensor>> weight_scale,
    std::optional<std::vector<torch::Tensor>> output_vec_scale, bool /*fast_accum*/, int64_t sm_margin,
    bool with_stream_sync) {
  return forward_impl(inputs, weights, splits_cpu, routing_idx, input_scale, weight_scale, output_vec_scale,
                      with_stream_sync, sm_margin);
}

// ------------------------------------------------------------------------------------------------
// Plain grouped GEMM
// ------------------------------------------------------------------------------------------------
GemmGroupedV3::GemmGroupedV3(torch::Tensor weight, int64_t num_experts) : weight_(weight) {
  to_fluxmi_dtype(weight.scalar_type());
  FLUX_AMD_CHECK_INPUT(weight, weight.scalar_type());
  TORCH_CHECK(weight.dim() == 3, "gemm grouped weight shape is not 3");
  TORCH_CHECK(weight.size(0) == num_experts, "gemm grouped 0-dim is not equal to num_experts");
}

torch::Tensor GemmGroupedV3::forward(torch::Tensor input, torch::Tensor splits_cpu) {
  FLUX_AMD_CHECK_INPUT(input, weight_.scalar_type());
  TORCH_CHECK(input.dim() == 2, "input shape is not 2");
  TORCH_CHECK(splits_cpu.dim() == 1, "splits_cpu shape is not 1");
  TORCH_CHECK(splits_cpu.scalar_type() == at::kInt || splits_cpu.scalar_type() == at::kLong,
              "splits_cpu type can be int or long");
  TORCH_CHECK(weight_.size(2) == input.size(1), "weight 2-dim mismatch: ", weight_.size(2), " != ", input.size(1));
  TORCH_CHECK(splits_cpu.size(0) == weight_.size(0), "splits 0-dim mismatch: ", splits_cpu.size(0), " != ",
              weight_.size(0));
  torch::Tensor out = torch::empty({input.size(0), weight_.size(1)}, input.options().dtype(moe_output_dtype(input.scalar_type())));
  if (input.size(0) == 0) return out;
  torch::Tensor splits_dev = splits_cpu.to(at::kInt).to(input.device(), /*non_blocking=*/true);
  run_grouped_gemm(input, weight_, splits_dev, out, nullptr, input.size(0), nullptr, nullptr, nullptr, nullptr, 0);
  return out;
}

}  // namespace flux_amd
