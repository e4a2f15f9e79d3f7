"""Host logic of the C++ op layer (flux_ths_pybind): names, signatures, defaults and argument errors.
Runs without a GPU: every check below fires before any kernel launch."""
import inspect

import pytest
import torch

import flux_amd


def test_module_exports_reference_names():
    m = flux_amd.flux_ths_pybind
    for name in ("MoeArguments", "DistEnvTPWithEP", "GemmGroupedV3AGScatter", "GemmGroupedV3GatherRS", "GemmGroupedV3",
                 "Quantization", "BlockScaleGemm", "calc_scatter_index", "topk_scatter_reduce", "bitwise_check",
                 "init_flux_shm", "uniform_initialize", "load_tuning_record", "ProfilingContext", "TuningRecord"):
        assert hasattr(m, name), name
        assert getattr(flux_amd, name) is getattr(m, name)
    for cls, methods in ((m.GemmGroupedV3AGScatter, ("forward", "forward_multiple_weights", "clear_buffers", "profiling")),
                         (m.GemmGroupedV3GatherRS, ("forward_gather_rs", "forward_gather_rs_multiple",
                                                    "forward_gather_rs_no_zerobuffer", "ep_zero_buffer", "profiling")),
                         (m.ProfilingContext, ("get_code", "get_all_prof_results", "get_latest_prof_result",
                                               "get_latest_record", "get_all_records")),
                         (m.BlockScaleGemm, ("forward", "forward_grouped", "forward_multistream", "reference", "profiling")),
                         (m.Quantization, ("quantize_vector_blockwise", "quantize_square_blockwise",
                                           "batch_quantize_square_blockwise"))):
        for meth in methods:
            assert hasattr(cls, meth), f"{cls.__name__}.{meth}"


def test_keyword_names_match_reference():
    m = flux_amd.flux_ths_pybind
    doc = m.GemmGroupedV3AGScatter.forward.__doc__
    for kw in ("inputs_shard", "weights", "splits_gpu", "scatter_index", "output_scale", "outputs_buf",
               "allgather_output", "fast_accum", "sm_margin"):
        assert kw in doc, kw
    doc = m.GemmGroupedV3GatherRS.forward_gather_rs.__doc__
    for kw in ("input", "weight", "splits_cpu", "routing_idx", "n_tokens_per_rank", "input_scale", "weight_scale",
               "output_vec_scale", "fast_accum", "sm_margin", "with_stream_sync"):
        assert kw in doc, kw
    assert "return_tranpose" in m.Quantization.quantize_vector_blockwise.__doc__  # the reference's spelling
    doc = m.BlockScaleGemm.forward_grouped.__doc__  # src/pybind/gemm_only.cc:130-139
    for kw in ("input", "input_splits", "weight", "bias", "output", "input_scale", "weight_scale"):
        assert kw in doc, kw
    for kw in ("input_dtype", "weight_dtype", "output_dtype", "num_streams"):
        assert kw in m.BlockScaleGemm.__init__.__doc__, kw
    doc = m.BlockScaleGemm.forward_multistream.__doc__  # src/pybind/gemm_only.cc:110-119
    for kw in ("input", "input_splits", "weight", "bias", "output", "input_scale", "weight_scale"):
        assert kw in doc, kw
    assert "is_groupwise_b" in m.BlockScaleGemm.reference.__doc__ and "prof_ctx" in m.BlockScaleGemm.profiling.__doc__
    doc = m.GemmGroupedV3GatherRS.__init__.__doc__
    for kw in ("total_num_experts", "max_m", "n_dim", "topk", "rank", "world_size", "tp_world_size", "ep_world_size",
               "max_input_groups", "ep_in_dp"):
        assert kw in doc, kw


def test_world_size_above_one_is_rejected():
    with pytest.raises(RuntimeError, match="one GPU only"):
        flux_amd.GemmGroupedV3GatherRS(8, 512, 1024, 2, 0, 2, 2, 1)
    with pytest.raises(RuntimeError, match="one GPU only"):
        flux_amd.GemmGroupedV3GatherRS(8, 512, 1024, 2, 0, 1, 1, 2)

    class FakeGroup:
        def __init__(self, n):
            self.n = n

        def size(self):
            return self.n

    flux_amd.DistEnvTPWithEP(FakeGroup(1), 1)
    flux_amd.DistEnvTPWithEP(None, 1, None)
    with pytest.raises(RuntimeError, match="world size 1"):
        flux_amd.DistEnvTPWithEP(FakeGroup(8), 1)
    with pytest.raises(RuntimeError, match="nnodes"):
        flux_amd.DistEnvTPWithEP(None, 2)
    flux_amd.init_flux_shm(None)
    with pytest.raises(TypeError):
        flux_amd.load_tuning_record(object())  # takes a TuningRecord (from a ProfilingContext)
    with pytest.raises(RuntimeError, match="unsupported dtype"):
        flux_amd.uniform_initialize(torch.zeros(4), 1, 0.0, 1.0)


def test_dtype_and_device_checks():
    with pytest.raises(RuntimeError, match="bfloat16"):
        flux_amd.Quantization(torch.float16, torch.float8_e4m3fn)
    with pytest.raises(RuntimeError, match="float8_e4m3fn"):
        flux_amd.Quantization(torch.bfloat16, torch.float8_e5m2)
    q = flux_amd.Quantization(torch.bfloat16, torch.float8_e4m3fn)
    with pytest.raises(RuntimeError, match="2 dimensions"):
        q.quantize_vector_blockwise(torch.zeros(4, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="device tensor"):
        q.quantize_vector_blockwise(torch.zeros(4, 8, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="2 dimensions"):
        q.quantize_square_blockwise(torch.zeros(2, 4, 8, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="device tensor"):
        q.quantize_square_blockwise(torch.zeros(4, 8, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="3 dimensions"):
        q.batch_quantize_square_blockwise(torch.zeros(4, 8, dtype=torch.bfloat16))
    args = flux_amd.MoeArguments(max_ntokens=16, hidden=64, ffn_hidden=128, nexperts=4, topk=2,
                                 input_dtype=torch.bfloat16)
    assert (args.max_ntokens, args.hidden, args.ffn_hidden, args.nexperts, args.topk) == (16, 64, 128, 4, 2)
    with pytest.raises(RuntimeError, match="unsupported dtype"):
        bad = flux_amd.MoeArguments(16, 64, 128, 4, 2, torch.float32)
        flux_amd.GemmGroupedV3AGScatter(flux_amd.DistEnvTPWithEP(None, 1), bad)
    with pytest.raises(RuntimeError, match="device tensor"):
        flux_amd.calc_scatter_index(torch.zeros(4, 2, dtype=torch.int32), torch.zeros(4, dtype=torch.int32))
    with pytest.raises(RuntimeError, match="device tensor"):
        flux_amd.topk_scatter_reduce([torch.zeros(8, 8, dtype=torch.bfloat16)], torch.zeros(8, dtype=torch.int32), 2)
    with pytest.raises(RuntimeError):
        flux_amd.GemmGroupedV3(torch.zeros(2, 8, 8, dtype=torch.bfloat16), 2)  # host weight
    assert flux_amd.bitwise_check(torch.arange(6).view(2, 3), torch.arange(6).view(2, 3))
    assert not flux_amd.bitwise_check(torch.zeros(3), torch.zeros(4))
    assert not flux_amd.bitwise_check(torch.tensor([0.0]), torch.tensor([-0.0]))


def test_tuning_text_round_trip_and_errors():
    """The shape-keyed schedule table: text in, records counted, malformed lines rejected with their line number."""
    m = flux_amd.flux_ths_pybind
    m.clear_tuning_records()
    text = ("# comment\n"
            "fluxmi_gemm_tuning dtype=bf16 experts=8 n=14336 k=4096 rows=16384 groups=1 raster_rows=16 sched_flags=1\n"
            "\n"
            "fluxmi_gemm_tuning dtype=e4m3 experts=32 n=7168 k=2048 rows=32768 groups=1 raster_rows=4 sched_flags=0  # x\n")
    assert m.load_tuning_text(text) == 2
    assert m.num_tuning_records() == 2
    assert m.load_tuning_text(text) == 2 and m.num_tuning_records() == 2   # same keys: replaced, not duplicated
    for bad, what in (("fluxmi_gemm_tuning dtype=bf16 experts=8", "missing fields"),
                      ("something else", "expected 'fluxmi_gemm_tuning'"),
                      ("fluxmi_gemm_tuning dtype=fp64 experts=1 n=1 k=1 rows=1 groups=1 raster_rows=1 sched_flags=0", "unknown dtype"),
                      ("fluxmi_gemm_tuning dtype=bf16 experts=x n=1 k=1 rows=1 groups=1 raster_rows=1 sched_flags=0", "bad number"),
                      ("fluxmi_gemm_tuning dtype=bf16 experts=1 n=1 k=1 rows=1 groups=1 raster_rows=1 sched_flags=64", "out of range")):
        with pytest.raises(RuntimeError, match=what):
            m.load_tuning_text("# first line\n" + bad)
    # fp16 shapes, the newer schedule flags and the form of layer1's reduction are part of the text form
    assert m.load_tuning_text("fluxmi_gemm_tuning dtype=f16 experts=8 n=4096 k=14336 rows=16384 groups=1 raster_rows=8 "
                              "sched_flags=8 reduce=fused\n"
                              "fluxmi_gemm_tuning dtype=bf16 experts=8 n=4096 k=14336 rows=16384 groups=1 raster_rows=8 "
                              "sched_flags=4 reduce=twopass\n") == 2
    # ... and so is the form of the MFMA kernel's ring fills (16 half lines, 32 whole lines)
    assert m.load_tuning_text("fluxmi_gemm_tuning dtype=e4m3 experts=32 n=2048 k=7168 rows=32768 groups=1 raster_rows=8 "
                              "sched_flags=32\n"
                              "fluxmi_gemm_tuning dtype=bf16 experts=8 n=4096 k=14336 rows=16384 groups=1 raster_rows=8 "
                              "sched_flags=16\n") == 2
    with pytest.raises(RuntimeError, match="unknown reduce form"):
        m.load_tuning_text("fluxmi_gemm_tuning dtype=bf16 experts=1 n=1 k=1 rows=1 groups=1 raster_rows=1 sched_flags=0 reduce=maybe")
    m.clear_tuning_records()
    assert m.num_tuning_records() == 0
    ctx = m.ProfilingContext("empty")
    assert "empty" in ctx.get_code() and ctx.get_all_records() == []
    with pytest.raises(RuntimeError, match="no latest prof results"):
        ctx.get_latest_record()
