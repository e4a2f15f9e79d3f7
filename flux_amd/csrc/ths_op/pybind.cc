// Python module `flux_ths_pybind`: the class / function names and keyword arguments of the reference's
// module of the same name (src/pybind/gemm_grouped_v3_ag_scatter.cc:29-68,
// src/pybind/gemm_grouped_v3_gather_rs.cc:36-127, src/pybind/quantization.cc:30-57, src/pybind/ths_op.cc:106-146,
// :206-211, :316-320) for the single-GPU MoE path.
#include <torch/csrc/utils/pybind.h>

#include "ths_ops.h"

namespace py = pybind11;
using namespace flux_amd;

static at::ScalarType to_dtype(const py::object &o) { return torch::python::detail::py_object_to_dtype(o); }

// tp_group / ep_group: None or a torch.distributed ProcessGroup of size 1.
static void require_single_rank_group(const py::object &group, const char *name) {
  if (group.is_none()) return;
  const int size = group.attr("size")().cast<int>();
  if (size != 1) {
    throw std::runtime_error(std::string("DistEnvTPWithEP: ") + name + " has " + std::to_string(size) +
                             " ranks; this build runs on one GPU only (world size 1)");
  }
}

PYBIND11_MODULE(flux_ths_pybind, m) {
  m.doc() = "MI355X implementation of Flux's single-GPU MoE operators";

  py::class_<MoeArguments>(m, "MoeArguments")
      .def(py::init([](int32_t max_ntokens, int32_t hidden, int32_t ffn_hidden, int32_t nexperts, int32_t topk,
                       py::object input_dtype, py::object output_dtype) {
             const at::ScalarType in = to_dtype(input_dtype);
             at::ScalarType out = output_dtype.is_none() ? in : to_dtype(output_dtype);
             if (output_dtype.is_none() && is_fp8(in)) out = at::kBFloat16;
             return MoeArguments{max_ntokens, hidden, ffn_hidden, nexperts, topk, in, out};
           }),
           py::arg("max_ntokens"), py::arg("hidden"), py::arg("ffn_hidden"), py::arg("nexperts"), py::arg("topk"),
           py::arg("input_dtype"), py::arg("output_dtype") = py::none())
      .def_readonly("max_ntokens", &MoeArguments::max_ntokens)
      .def_readonly("hidden", &MoeArguments::hidden)
      .def_readonly("ffn_hidden", &MoeArguments::ffn_hidden)
      .def_readonly("nexperts", &MoeArguments::nexperts)
      .def_readonly("topk", &MoeArguments::topk);

  py::class_<DistEnvTPWithEP>(m, "DistEnvTPWithEP")
      .def(py::init([](py::object tp_group, int32_t nnodes, py::object ep_group) {
             require_single_rank_group(tp_group, "tp_group");
             require_single_rank_group(ep_group, "ep_group");
             if (nnodes != 1) throw std::runtime_error("DistEnvTPWithEP: nnodes must be 1 in this build");
             return DistEnvTPWithEP{};
           }),
           py::arg("tp_group") = py::none(), py::arg("nnodes") = 1, py::arg("ep_group") = py::none())
      .def("__repr__", &DistEnvTPWithEP::to_string);

  // src/pybind/ths_op.cc:78-92 (ProfilingContext, TuningRecord)
  py::class_<ProfilingContext, std::shared_ptr<ProfilingContext>>(m, "ProfilingContext")
      .def(py::init<std::string>(), py::arg("name"))
      .def("get_code", &ProfilingContext::get_code)
      .def("get_all_prof_results", &ProfilingContext::get_all_prof_results)
      .def("get_latest_prof_result", &ProfilingContext::get_latest_prof_result)
      .def("get_latest_record", &ProfilingContext::get_latest_record)
      .def("get_all_records", &ProfilingContext::get_all_records);
  py::class_<TuningRecord>(m, "TuningRecord")
      .def("__repr__", &TuningRecord::to_string)
      .def_property_readonly("shape", [](const TuningRecord &r) { return r.key.to_string(); })
      .def_property_readonly("raster_rows", [](const TuningRecord &r) { return r.best.raster_rows; })
      .def_property_readonly("sched_flags", [](const TuningRecord &r) { return r.best.sched_flags; })
      .def_property_readonly("reduce_fused", [](const TuningRecord &r) { return r.best.reduce_fused != 0; });

  py::class_<GemmGroupedV3AGScatter>(m, "GemmGroupedV3AGScatter")
      .def(py::init<DistEnvTPWithEP, MoeArguments>(), py::arg("tp_env"), py::arg("moe_args"))
      .def("clear_buffers", &GemmGroupedV3AGScatter::clear_buffers)
      .def("forward", &GemmGroupedV3AGScatter::forward, py::arg("inputs_shard"), py::arg("weights"),
           py::arg("splits_gpu"), py::arg("scatter_index"), py::arg("output_scale") = py::none(),
           py::arg("outputs_buf") = py::none(), py::arg("allgather_output") = py::none(),
           py::arg("fast_accum") = false, py::arg("sm_margin") = 0)
      .def("forward_multiple_weights", &GemmGroupedV3AGScatter::forward_multiple_weights, py::arg("inputs_shard"),
           py::arg("weights"), py::arg("splits_gpu"), py::arg("scatter_index"), py::arg("output_scale") = py::none(),
           py::arg("outputs_buf") = py::none(), py::arg("allgather_output") = py::none(),
           py::arg("fast_accum") = false, py::arg("sm_margin") = 0)
      .def("profiling", &GemmGroupedV3AGScatter::profiling, py::arg("inputs_shard"), py::arg("weights"),
           py::arg("splits_gpu"), py::arg("scatter_index"), py::arg("output_scale") = py::none(),
           py::arg("outputs_buf") = py::none(), py::arg("allgather_output") = py::none(),
           py::arg("fast_accum") = false, py::arg("sm_margin") = 0, py::arg("prof_ctx") = nullptr);

  py::class_<GemmGroupedV3GatherRS>(m, "GemmGroupedV3GatherRS")
      // The reference's ten arguments (src/pybind/gemm_grouped_v3_gather_rs.cc:36-50) and, after them, one of this
      // build: the dtype of the [M, N] intermediate between the GEMM and the top-k reduction.  None / torch.float32
      // (default): one rounding in the whole layer; the 16-bit output type (torch.bfloat16 / torch.float16): the
      // reference's own data flow (its inter_D), each top-k term rounded before the sum, half the intermediate's
      // bytes, the reference's own 2e-2 test bound.  $FLUX_AMD_INTER_DTYPE=bf16 sets the default to the latter.
      .def(py::init([](int64_t total_num_experts, int64_t max_m, int64_t n_dim, int64_t topk, int64_t rank,
                       int64_t world_size, int64_t tp_world_size, int64_t ep_world_size, int64_t max_input_groups,
                       bool ep_in_dp, py::object inter_dtype) {
             auto *op = new GemmGroupedV3GatherRS(total_num_experts, max_m, n_dim, topk, rank, world_size, tp_world_size,
                                                  ep_world_size, max_input_groups, ep_in_dp);
             if (!inter_dtype.is_none()) {
               const at::ScalarType t = to_dtype(inter_dtype);
               if (t != at::kFloat && t != at::kBFloat16 && t != at::kHalf) {
                 delete op;
                 TORCH_CHECK(false, "inter_dtype must be torch.float32 or the 16-bit output type, got ", t);
               }
               op->set_intermediate_fp32(t == at::kFloat);
             }
             return op;
           }),
           py::arg("total_num_experts"), py::arg("max_m"), py::arg("n_dim"), py::arg("topk"), py::arg("rank"),
           py::arg("world_size"), py::arg("tp_world_size"), py::arg("ep_world_size"),
           py::arg("max_input_groups") = 1, py::arg("ep_in_dp") = false, py::arg("inter_dtype") = py::none())
      .def("forward_gather_rs", &GemmGroupedV3GatherRS::forward_gather_rs, py::arg("input"), py::arg("weight"),
           py::arg("splits_cpu"), py::arg("routing_idx"), py::arg("n_tokens_per_rank") = py::none(),
           py::arg("input_scale") = py::none(), py::arg("weight_scale") = py::none(),
           py::arg("output_vec_scale") = py::none(), py::arg("fast_accum") = false, py::arg("sm_margin") = 0,
           py::arg("with_stream_sync") = false)
      .def("forward_gather_rs_no_zerobuffer", &GemmGroupedV3GatherRS::forward_gather_rs, py::arg("input"),
           py::arg("weight"), py::arg("splits_cpu"), py::arg("routing_idx"), py::arg("n_tokens_per_rank") = py::none(),
           py::arg("input_scale") = py::none(), py::arg("weight_scale") = py::none(),
           py::arg("output_vec_scale") = py::none(), py::arg("fast_accum") = false, py::arg("sm_margin") = 0,
           py::arg("with_stream_sync") = false)
      .def("forward_gather_rs_multiple", &GemmGroupedV3GatherRS::forward_gather_rs_multiple, py::arg("input"),
           py::arg("weight"), py::arg("splits_cpu"), py::arg("routing_idx"), py::arg("n_tokens_per_rank") = py::none(),
           py::arg("input_scale") = py::none(), py::arg("weight_scale") = py::none(),
           py::arg("output_vec_scale") = py::none(), py::arg("fast_accum") = true, py::arg("sm_margin") = 0,
           py::arg("with_stream_sync") = false)
      .def("ep_zero_buffer", &GemmGroupedV3GatherRS::ep_zero_buffer)
      .def("profiling", &GemmGroupedV3GatherRS::profiling, py::arg("input"), py::arg("weight"), py::arg("splits_cpu"),
           py::arg("routing_idx"), py::arg("n_tokens_per_rank") = py::none(), py::arg("input_scale") = py::none(),
           py::arg("weight_scale") = py::none(), py::arg("output_vec_scale") = py::none(),
           py::arg("fast_accum") = false, py::arg("sm_margin") = 0, py::arg("with_stream_sync") = false,
           py::arg("prof_ctx") = nullptr);

  py::class_<GemmGroupedV3>(m, "GemmGroupedV3")
      .def(py::init<torch::Tensor, int64_t>(), py::arg("weight"), py::arg("num_experts"))
      .def("forward", &GemmGroupedV3::forward, py::arg("input"), py::arg("splits_cpu"));

  // src/pybind/gemm_only.cc:77-139 (forward, forward_grouped, forward_multistream, reference, profiling; only the
  // weight-gradient methods wgrad* are absent)
  py::class_<BlockScaleGemm>(m, "BlockScaleGemm")
      .def(py::init([](py::object input_dtype, py::object weight_dtype, py::object output_dtype, int32_t num_streams) {
             const at::ScalarType in = to_dtype(input_dtype);
             return new BlockScaleGemm(in, to_dtype(weight_dtype), output_dtype.is_none() ? in : to_dtype(output_dtype),
                                       num_streams);
           }),
           py::arg("input_dtype"), py::arg("weight_dtype"), py::arg("output_dtype") = py::none(),
           py::arg("num_streams") = 2)
      .def("forward", &BlockScaleGemm::forward, py::arg("input"), py::arg("weight"), py::arg("bias") = py::none(),
           py::arg("output") = py::none(), py::arg("input_scale") = py::none(), py::arg("weight_scale") = py::none())
      .def("forward_grouped", &BlockScaleGemm::forward_grouped, py::arg("input"), py::arg("input_splits"),
           py::arg("weight"), py::arg("bias") = py::none(), py::arg("output") = py::none(),
           py::arg("input_scale") = py::none(), py::arg("weight_scale") = py::none())
      .def("forward_multistream", &BlockScaleGemm::forward_multistream, py::arg("input"), py::arg("input_splits"),
           py::arg("weight"), py::arg("bias") = py::none(), py::arg("output") = py::none(),
           py::arg("input_scale") = py::none(), py::arg("weight_scale") = py::none())
      .def("reference", &BlockScaleGemm::reference, py::arg("input"), py::arg("weight"), py::arg("bias") = py::none(),
           py::arg("output") = py::none(), py::arg("input_scale") = py::none(), py::arg("weight_scale") = py::none(),
           py::arg("is_groupwise_b") = false)
      .def("profiling", &BlockScaleGemm::profiling, py::arg("input"), py::arg("weight"), py::arg("bias") = py::none(),
           py::arg("output") = py::none(), py::arg("input_scale") = py::none(), py::arg("weight_scale") = py::none(),
           py::arg("prof_ctx") = nullptr);

  py::class_<Quantization>(m, "Quantization")
      .def(py::init([](py::object input_dtype, py::object output_dtype, int32_t num_streams) {
             return new Quantization(to_dtype(input_dtype), to_dtype(output_dtype), num_streams);
           }),
           py::arg("input_dtype"), py::arg("output_dtype"), py::arg("num_streams") = 2)
      // "return_tranpose" is the reference's own spelling of the keyword (src/pybind/quantization.cc:45).
      .def("quantize_vector_blockwise", &Quantization::quantize_vector_blockwise, py::arg("input"),
           py::arg("return_tranpose") = true, py::arg("eps") = 0.0)
      .def("quantize_square_blockwise", &Quantization::quantize_square_blockwise, py::arg("input"),
           py::arg("return_tranpose") = true, py::arg("eps") = 0.0)
      .def("batch_quantize_square_blockwise", &Quantization::batch_quantize_square_blockwise, py::arg("input"),
           py::arg("return_tranpose") = true, py::arg("eps") = 0.0)
      .def("quantize_rowwise", &Quantization::quantize_rowwise, py::arg("input"), py::arg("eps") = 0.0);

  m.def("calc_scatter_index", &calc_scatter_index, py::arg("choosed_experts"), py::arg("splits"));
  m.def("moe_route_sort", &moe_route_sort, py::arg("choosed_experts"), py::arg("nexperts"));
  m.def("topk_scatter_reduce", &topk_scatter_reduce, py::arg("inputs"), py::arg("scatter_idx"), py::arg("TOPK"));
  m.def("topk_weighted_gather_reduce", &topk_weighted_gather_reduce, py::arg("inputs"), py::arg("routing_idx"),
        py::arg("topk"), py::arg("row_weight") = py::none(), py::arg("scale") = 1.0);
  m.def("bitwise_check", &bitwise_check);
  m.def("init_flux_shm", [](py::object) {}, py::arg("group") = py::none());  // nothing to set up on one GPU
  // Test helper of the reference (src/ths_op/helper_ops.cc:33-44, src/cuda/random_initialize.cu:27-51): fills a
  // half / bf16 / fp8 device tensor with uniform values of [min, max] from `seed`.  The values come from torch's
  // generator, not from cuRAND's: the same seed gives the same tensor here, not the reference's tensor.
  m.def("uniform_initialize", [](torch::Tensor tensor, uint64_t seed, double min, double max) {
    const at::ScalarType st = tensor.scalar_type();
    TORCH_CHECK(st == at::kHalf || st == at::kBFloat16 || st == at::ScalarType::Float8_e4m3fn ||
                    st == at::ScalarType::Float8_e5m2,
                "unsupported dtype: ", st);
    TORCH_CHECK(tensor.is_cuda(), "uniform_initialize: tensor must be a device tensor");
    py::object torch_mod = py::module_::import("torch");
    py::object gen = torch_mod.attr("Generator")(py::arg("device") = tensor.device().str());
    gen.attr("manual_seed")(seed);
    py::object tmp = torch_mod.attr("empty")(tensor.sizes().vec(), py::arg("dtype") = torch_mod.attr("float32"),
                                            py::arg("device") = tensor.device().str());
    tmp.attr("uniform_")(min, max, py::arg("generator") = gen);
    tensor.copy_(tmp.cast<torch::Tensor>());
    return true;
  });
  // The reference's tuning records select among its generated kernel variants (src/ths_op/ths_op.cc:213-216);
  // here a record selects the tile schedule of the persistent grouped GEMM for one problem shape.
  m.def("load_tuning_record", [](const TuningRecord &r) { TuningTable::instance().add(r.key, r.best); },
        py::arg("record"));
  // Text written by ProfilingContext.get_code(); also read once per process from $FLUX_AMD_TUNING_FILE.
  m.def("load_tuning_text", [](const std::string &text) { return TuningTable::instance().load_text(text); },
        py::arg("text"));
  m.def("clear_tuning_records", []() { TuningTable::instance().clear(); });
  m.def("num_tuning_records", []() { return TuningTable::instance().size(); });
}
