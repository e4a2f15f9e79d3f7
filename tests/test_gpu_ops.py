"""GPU parity through the operator surface (flux_ths_pybind), written the way the reference's own tests use the
ops: build the op, call forward, compare with the torch layer (test/python/moe_ag_scatter/test_moe_ag.py:213-311,
:544-565; test/python/moe_gather_rs/test_moe_gather_rs.py:210-298, :635-648; chaining as in
examples/moe_flux_only.py:112-131).  bf16 bound: rtol 1e-2 / atol 1e-2 against the fp32 oracle."""
import numpy as np
import pytest
import torch

import flux_amd
from oracle import configs, layers, quant, routing

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-2, 1e-2


def close(got, ref):
    got = got.float().cpu()
    bad = (got - ref).abs() > ATOL + RTOL * ref.abs()
    assert not bool(bad.any()), f"{int(bad.sum())} of {bad.numel()} outside tolerance, max {float((got - ref).abs().max())}"


@pytest.fixture(scope="module")
def c1():
    return configs.make_workload("C1")


def test_routing_functions(c1):
    wl = c1
    choosed = wl.choosed.cuda()
    splits, scatter, gather, tki = flux_amd.moe_route_sort(choosed, wl.experts)
    assert np.array_equal(splits.cpu().numpy(), wl.splits)
    assert np.array_equal(scatter.cpu().numpy(), wl.scatter_index)
    assert np.array_equal(gather.cpu().numpy(), wl.gather_index)
    assert np.array_equal(tki.cpu().numpy(), wl.topk_index)
    s2 = flux_amd.calc_scatter_index(choosed, splits)
    assert flux_amd.bitwise_check(s2, scatter)
    assert routing.is_gather_index_stable(gather.cpu().numpy(), wl.splits)


def test_layer0_layer1_chain_c1(c1):
    """layer0 forward(outputs_buf=intermediate) -> layer1 forward_gather_rs(routing_idx=scatter_index.view(-1))."""
    wl = c1
    t, k, e, h, f = wl.tokens, wl.topk, wl.experts, wl.hidden, wl.ffn
    x, w1, w2 = (wl.tensors[n].cuda() for n in ("x", "w1", "w2"))
    splits_gpu = torch.from_numpy(wl.splits).cuda()
    scatter_index = torch.from_numpy(wl.scatter_index).cuda()
    tp_env = flux_amd.DistEnvTPWithEP(tp_group=None, nnodes=1, ep_group=None)
    moe_args = flux_amd.MoeArguments(max_ntokens=t, hidden=h, ffn_hidden=f, nexperts=e, topk=k,
                                     input_dtype=torch.bfloat16)
    op0 = flux_amd.GemmGroupedV3AGScatter(tp_env=tp_env, moe_args=moe_args)
    inter = torch.empty(t * k, f, dtype=torch.bfloat16, device="cuda")
    ag = torch.empty_like(x)
    op0.clear_buffers()
    out0 = op0.forward(inputs_shard=x, weights=w1, splits_gpu=splits_gpu, scatter_index=scatter_index,
                       outputs_buf=inter, allgather_output=ag, fast_accum=False, sm_margin=0)
    assert out0.data_ptr() == inter.data_ptr()
    assert torch.equal(ag, x)
    close(out0, layers.layer0_fp32(wl.tensors["x"], wl.tensors["w1"], wl.splits, wl.gather_index))
    # with output_scale; fresh output tensor
    alpha = (torch.rand(e) + 0.5)
    out0s = op0.forward(x, w1, splits_gpu, scatter_index, output_scale=alpha.cuda())
    close(out0s, layers.layer0_fp32(wl.tensors["x"], wl.tensors["w1"], wl.splits, wl.gather_index, alpha))
    # the reference's own op order (two bf16 roundings) stays within its own bound, 1e-2 / 1.5e-2
    ref_t = layers.layer0_torch(wl.tensors["x"], wl.tensors["w1"], wl.splits, wl.gather_index, alpha).float()
    assert torch.allclose(out0s.float().cpu(), ref_t, atol=1e-2, rtol=1.5e-2)

    op1 = flux_amd.GemmGroupedV3GatherRS(total_num_experts=e, max_m=t * k, n_dim=h, topk=k, rank=0, world_size=1,
                                         tp_world_size=1, ep_world_size=1, max_input_groups=2)
    splits_cpu = torch.from_numpy(wl.splits)
    ovs = wl.row_weight.cuda()
    out1 = op1.forward_gather_rs(input=inter, weight=w2, splits_cpu=splits_cpu, routing_idx=scatter_index.view(-1),
                                 output_vec_scale=ovs)
    assert out1.shape == (t, h) and out1.dtype == torch.bfloat16
    ref1 = layers.layer1_fp32(inter.cpu(), wl.tensors["w2"], wl.splits, wl.scatter_index.reshape(-1), k,
                              output_vec_scale=wl.row_weight)
    close(out1, ref1)
    # scalar input_scale [1] and per-expert weight_scale [E]
    s_in, s_w = torch.tensor([0.75]), torch.rand(e) + 0.5
    out1s = op1.forward_gather_rs(inter, w2, splits_cpu, scatter_index.view(-1), input_scale=s_in.cuda(),
                                  weight_scale=s_w.cuda(), output_vec_scale=ovs, with_stream_sync=True)
    close(out1s, layers.layer1_fp32(inter.cpu(), wl.tensors["w2"], wl.splits, wl.scatter_index.reshape(-1), k,
                                    s_in, s_w, wl.row_weight))
    # two input groups are summed before the reduce
    out2 = op1.forward_gather_rs_multiple([inter, inter], [w2, w2], splits_cpu, scatter_index.view(-1),
                                          output_vec_scale=[ovs, ovs])
    close(out2, 2 * ref1)


def test_forward_multiple_weights_and_plain_grouped_gemm(c1):
    wl = c1
    x, w1 = wl.tensors["x"].cuda(), wl.tensors["w1"].cuda()
    w1b = (w1.float() * 0.5).to(torch.bfloat16)
    op0 = flux_amd.GemmGroupedV3AGScatter(flux_amd.DistEnvTPWithEP(None, 1),
                                          flux_amd.MoeArguments(wl.tokens, wl.hidden, wl.ffn, wl.experts, wl.topk,
                                                                torch.bfloat16))
    outs = op0.forward_multiple_weights(x, [w1, w1b], torch.from_numpy(wl.splits).cuda(),
                                        torch.from_numpy(wl.scatter_index).cuda())
    ref = layers.layer0_fp32(wl.tensors["x"], wl.tensors["w1"], wl.splits, wl.gather_index)
    close(outs[0], ref)
    close(outs[1], 0.5 * ref)
    xs = x[torch.from_numpy(wl.gather_index).long().cuda()].contiguous()
    plain = flux_amd.GemmGroupedV3(w1, wl.experts).forward(xs, torch.from_numpy(wl.splits))
    assert torch.equal(plain, outs[0])  # same kernel, gather folded in or not: identical bits


def test_topk_scatter_reduce_and_shape_errors(c1):
    wl = c1
    g = torch.Generator().manual_seed(3)
    inter = torch.randn(wl.rows, 512, generator=g).to(torch.bfloat16)
    idx = torch.from_numpy(wl.scatter_index.reshape(-1))
    out = flux_amd.topk_scatter_reduce([inter.cuda(), inter.cuda()], idx.cuda(), wl.topk)
    close(out, layers.topk_gather_reduce_fp32([inter, inter], idx.numpy(), wl.topk))
    op1 = flux_amd.GemmGroupedV3GatherRS(wl.experts, wl.rows, wl.hidden, wl.topk, 0, 1, 1, 1)
    act, w2 = wl.tensors["act"].cuda(), wl.tensors["w2"].cuda()
    with pytest.raises(RuntimeError, match="host tensor"):
        op1.forward_gather_rs(act, w2, torch.from_numpy(wl.splits).cuda(), idx.cuda())
    with pytest.raises(RuntimeError, match="splits 0-dim mismatch"):
        op1.forward_gather_rs(act, w2, torch.zeros(3, dtype=torch.int32), idx.cuda())
    with pytest.raises(RuntimeError, match="routing_idx"):
        op1.forward_gather_rs(act, w2, torch.from_numpy(wl.splits), idx[:-2].cuda())


def test_quantization_op():
    q = flux_amd.Quantization(torch.bfloat16, torch.float8_e4m3fn)
    g = torch.Generator().manual_seed(9)
    x = (torch.randn(200, 384, generator=g) * 3).to(torch.bfloat16)
    bits = x.view(torch.int16).numpy().view(np.uint16)
    out, scale, out_t, scale_t = q.quantize_vector_blockwise(x.cuda(), return_tranpose=True)
    rq, rs = quant.quant_rows_c(bits, 128, 0.0, True)
    assert out.dtype == torch.float8_e4m3fn and tuple(scale.shape) == (2, 3, 128)
    assert np.array_equal(out.view(torch.uint8).cpu().numpy(), rq) and np.array_equal(scale.cpu().numpy(), rs)
    bits_t = np.ascontiguousarray(bits.T)
    rqt, rst = quant.quant_rows_c(bits_t, 128, 0.0, True)
    assert tuple(out_t.shape) == (384, 200) and tuple(scale_t.shape) == (3, 2, 128)
    assert np.array_equal(out_t.view(torch.uint8).cpu().numpy(), rqt) and np.array_equal(scale_t.cpu().numpy(), rst)
    out2, scale2, none_t, none_s = q.quantize_vector_blockwise(x.cuda(), return_tranpose=False)
    assert none_t is None and none_s is None and torch.equal(out2.view(torch.uint8), out.view(torch.uint8))
    qr, sr = q.quantize_rowwise(x.cuda())
    rq0, rs0 = quant.quant_rows_c(bits)
    assert np.array_equal(qr.view(torch.uint8).cpu().numpy(), rq0) and np.array_equal(sr.cpu().numpy(), rs0)


def test_uniform_initialize():
    for dt in (torch.bfloat16, torch.float16, torch.float8_e4m3fn):
        t = torch.zeros(4096, dtype=dt, device="cuda")
        assert flux_amd.uniform_initialize(t, 7, -0.5, 1.5)
        f = t.float()
        assert float(f.min()) >= -0.5 and float(f.max()) <= 1.5 and 0.3 < float(f.mean()) < 0.7
        u = torch.zeros(4096, dtype=dt, device="cuda")
        flux_amd.uniform_initialize(u, 7, -0.5, 1.5)
        assert torch.equal(t.view(torch.uint8), u.view(torch.uint8))
        flux_amd.uniform_initialize(u, 8, -0.5, 1.5)
        assert not torch.equal(t.view(torch.uint8), u.view(torch.uint8))


def test_quantization_square_ops():
    """quantize_square_blockwise / batch_quantize_square_blockwise: shapes, dtypes and values of the four results."""
    q = flux_amd.Quantization(torch.bfloat16, torch.float8_e4m3fn)
    g = torch.Generator().manual_seed(10)
    x = (torch.randn(3, 200, 384, generator=g) * 3).to(torch.bfloat16)
    bits = x.view(torch.int16).numpy().view(np.uint16)
    out, scale, out_t, scale_t = q.quantize_square_blockwise(x[0].cuda(), return_tranpose=True)
    rq, rs = quant.quant_square_c(bits[0])
    assert out.dtype == torch.float8_e4m3fn and tuple(out.shape) == (200, 384) and tuple(scale.shape) == (2, 3)
    assert tuple(out_t.shape) == (384, 200) and tuple(scale_t.shape) == (3, 2)
    assert np.array_equal(out.view(torch.uint8).cpu().numpy(), rq) and np.array_equal(scale.cpu().numpy(), rs)
    assert np.array_equal(out_t.view(torch.uint8).cpu().numpy(), rq.T) and np.array_equal(scale_t.cpu().numpy(), rs.T)
    out2, scale2, none_t, none_s = q.quantize_square_blockwise(x[0].cuda(), return_tranpose=False)
    assert none_t is None and none_s is None and torch.equal(out2.view(torch.uint8), out.view(torch.uint8))
    bo, bs, bot, bst = q.batch_quantize_square_blockwise(x.cuda())  # transposed outputs by default
    assert tuple(bo.shape) == (3, 200, 384) and tuple(bs.shape) == (3, 2, 3)
    assert tuple(bot.shape) == (3, 384, 200) and tuple(bst.shape) == (3, 3, 2)
    for b in range(3):
        rq, rs = quant.quant_square_c(bits[b])
        assert np.array_equal(bo[b].view(torch.uint8).cpu().numpy(), rq) and np.array_equal(bs[b].cpu().numpy(), rs)
        assert np.array_equal(bot[b].view(torch.uint8).cpu().numpy(), rq.T) and np.array_equal(bst[b].cpu().numpy(), rs.T)


def test_fp8_layer1_through_ops():
    """fp8 activations and weights with per-row x per-output-channel scales (weight_scale [E, N], input_scale [M])."""
    wl = configs.make_workload("C5", tokens=128, hidden=512, ffn=256)
    e, k = wl.experts, wl.topk
    q = flux_amd.Quantization(torch.bfloat16, torch.float8_e4m3fn)
    act, w2 = wl.tensors["act"].cuda(), wl.tensors["w2"].cuda()
    qa, sa = q.quantize_rowwise(act)
    qw, sw = q.quantize_rowwise(w2.reshape(-1, wl.ffn))
    qw, sw = qw.reshape(e, wl.hidden, wl.ffn), sw.reshape(e, wl.hidden)
    op1 = flux_amd.GemmGroupedV3GatherRS(e, wl.rows, wl.hidden, k, 0, 1, 1, 1)
    out = op1.forward_gather_rs(qa, qw, torch.from_numpy(wl.splits), torch.from_numpy(wl.scatter_index.reshape(-1)).cuda(),
                                input_scale=sa, weight_scale=sw, output_vec_scale=wl.row_weight.cuda(), fast_accum=True)
    z = layers.fp8_grouped_gemm_fp32(qa.cpu(), sa.cpu(), qw.cpu(), sw.cpu(), wl.splits, row_weight=wl.row_weight)
    ref = layers.topk_gather_reduce_fp32(z, wl.scatter_index.reshape(-1), k)
    err = float((out.float().cpu() - ref).norm() / ref.norm())
    assert err < 3e-2, err


def test_fp8_c5_chain_through_ops_full_size():
    """C5 at full size through the operator classes, the reference's call sequence (examples/moe_flux_only.py:112-131):
    layer0 GemmGroupedV3AGScatter on e4m3 tokens and weights with the reference's fp8 scale form (one activation
    scale, one scale per expert, folded into output_scale [E]; python/flux/cpp_mod.pyi:932-938), its bf16 output
    quantised per row, layer1 GemmGroupedV3GatherRS with input_scale [M] x weight_scale [E, N] and the top-8
    weights as output_vec_scale.  Sampled rows / tokens against the dequantise-matmul oracle on the same bytes."""
    wl = configs.make_workload("C5")
    t, k, e, h, f, m = wl.tokens, wl.topk, wl.experts, wl.hidden, wl.ffn, wl.rows
    print(f"[case] ops chain fp8 C5 T={t} k={k} E={e} H={h} F={f}", flush=True)
    rng = np.random.default_rng(73)
    q = flux_amd.Quantization(torch.bfloat16, torch.float8_e4m3fn)
    x, w1, w2 = (wl.tensors[n].cuda() for n in ("x", "w1", "w2"))
    # layer0 operands: per-tensor activation scale, per-expert weight scale
    sx = float(x.float().abs().max()) / 448.0
    qx = (x.float() / sx).to(torch.float8_e4m3fn)
    sw1 = w1.float().abs().amax(dim=(1, 2)) / 448.0
    qw1 = (w1.float() / sw1[:, None, None]).to(torch.float8_e4m3fn)
    output_scale = (sw1 * sx).contiguous()
    splits_gpu = torch.from_numpy(wl.splits).cuda()
    scatter_index = torch.from_numpy(wl.scatter_index).cuda()
    op0 = flux_amd.GemmGroupedV3AGScatter(flux_amd.DistEnvTPWithEP(None, 1, None),
                                          flux_amd.MoeArguments(t, h, f, e, k, torch.float8_e4m3fn, torch.bfloat16))
    y = op0.forward(qx, qw1, splits_gpu, scatter_index, output_scale=output_scale, fast_accum=False)
    assert y.dtype == torch.bfloat16 and tuple(y.shape) == (m, f)
    eor = routing.expert_of_row(wl.splits)
    off = routing.offsets(wl.splits)
    rows = np.concatenate([np.array([off[i], off[i + 1] - 1]) for i in range(e) if off[i + 1] > off[i]]
                          + [rng.integers(0, m, size=64)])
    qx_c, qw1_c, os_c = qx.cpu().float(), qw1.cpu(), output_scale.cpu()
    for r in rows:
        ee = int(eor[r])
        ref = (qx_c[int(wl.gather_index[r])] @ qw1_c[ee].float().t()) * float(os_c[ee])
        got = y[int(r)].float().cpu()
        assert torch.allclose(got, ref, rtol=1e-2, atol=1e-2 * float(ref.abs().max())), f"layer0 row {r}"
    # layer1: per-row activation scales, per-output-channel weight scales
    qa, sa = q.quantize_rowwise(y)
    qw2, sw2 = q.quantize_rowwise(w2.reshape(-1, f))
    qw2, sw2 = qw2.reshape(e, h, f), sw2.reshape(e, h)
    op1 = flux_amd.GemmGroupedV3GatherRS(e, m, h, k, 0, 1, 1, 1)
    out = op1.forward_gather_rs(qa, qw2, torch.from_numpy(wl.splits), scatter_index.view(-1), input_scale=sa,
                                weight_scale=sw2, output_vec_scale=wl.row_weight.cuda(), fast_accum=False)
    assert out.dtype == torch.bfloat16 and tuple(out.shape) == (t, h)
    qa_c, sa_c, qw2_c, sw2_c = qa.cpu(), sa.cpu(), qw2.cpu(), sw2.cpu()
    tok = rng.integers(0, t, size=12)
    ref1 = torch.zeros(len(tok), h)
    for i, tt in enumerate(tok):
        for j in range(k):
            r = int(wl.scatter_index[tt, j])
            ee = int(eor[r])
            ref1[i] += float(wl.row_weight[r]) * float(sa_c[r]) * ((qa_c[r].float() @ qw2_c[ee].float().t()) * sw2_c[ee])
    got = out[torch.as_tensor(tok).cuda()].float().cpu()
    assert float((got - ref1).norm() / ref1.norm()) < 3e-2
    assert torch.allclose(got, ref1, rtol=1e-2, atol=1e-2 * float(ref1.abs().max()))


def test_profiling_registers_a_schedule_and_keeps_results(c1):
    """profiling() of both layer ops: every tile schedule gives the bits of forward(); the fastest is recorded in
    the context, registered for the shape, and its text form loads back."""
    wl = c1
    m = flux_amd.flux_ths_pybind
    m.clear_tuning_records()
    t, k, e, h, f = wl.tokens, wl.topk, wl.experts, wl.hidden, wl.ffn
    x, w1, w2 = (wl.tensors[n].cuda() for n in ("x", "w1", "w2"))
    splits_gpu = torch.from_numpy(wl.splits).cuda()
    scatter_index = torch.from_numpy(wl.scatter_index).cuda()
    op0 = flux_amd.GemmGroupedV3AGScatter(flux_amd.DistEnvTPWithEP(None, 1, None),
                                          flux_amd.MoeArguments(t, h, f, e, k, torch.bfloat16))
    ref0 = op0.forward(x, w1, splits_gpu, scatter_index)
    ctx = flux_amd.ProfilingContext("c1")
    out0 = op0.profiling(x, w1, splits_gpu, scatter_index, prof_ctx=ctx)
    assert torch.equal(out0, ref0)
    assert m.num_tuning_records() == 1
    rec = ctx.get_latest_record()
    assert f"experts={e} n={f} k={h} rows={t * k} groups=1" in rec.shape
    assert rec.raster_rows in (4, 8, 16) and rec.sched_flags in (0, 1, 2, 3, 4, 8, 16, 32)
    assert ctx.get_latest_prof_result().count("TopK=") == 5
    assert torch.equal(op0.forward(x, w1, splits_gpu, scatter_index), ref0)  # now under the registered schedule

    op1 = flux_amd.GemmGroupedV3GatherRS(e, t * k, h, k, 0, 1, 1, 1)
    routing_idx = scatter_index.view(-1)
    ref1 = op1.forward_gather_rs(ref0, w2, torch.from_numpy(wl.splits), routing_idx)
    out1 = op1.profiling(ref0, w2, torch.from_numpy(wl.splits), routing_idx, prof_ctx=ctx)
    assert torch.equal(out1, ref1)
    assert m.num_tuning_records() == 2 and len(ctx.get_all_records()) == 2 and len(ctx.get_all_prof_results()) == 2
    code = ctx.get_code()
    assert code.count("fluxmi_gemm_tuning") == 2
    m.clear_tuning_records()
    assert m.load_tuning_text(code) == 2
    m.clear_tuning_records()
    m.load_tuning_record(rec)
    assert m.num_tuning_records() == 1
    m.clear_tuning_records()
    # the layer1 record also says which form of the top-k reduction won; the text form carries it and loads back
    rec1 = ctx.get_latest_record()
    assert rec1.reduce_fused in (False, True)
    assert ("reduce=fused" in ctx.get_code().splitlines()[-1]) == rec1.reduce_fused
    assert m.load_tuning_text("fluxmi_gemm_tuning dtype=bf16 experts=%d n=%d k=%d rows=%d groups=1 raster_rows=8 "
                              "sched_flags=0 reduce=fused\n" % (e, h, f, t * k)) == 1
    forced = op1.forward_gather_rs(ref0, w2, torch.from_numpy(wl.splits), routing_idx)  # now the fused form
    assert torch.equal(forced, ref1)  # top-2: same bits either way
    m.clear_tuning_records()
    # without a context the profiler still runs and registers
    op0.profiling(x, w1, splits_gpu, scatter_index)
    assert m.num_tuning_records() == 1
    m.clear_tuning_records()


@pytest.mark.parametrize("raster_rows,flags,margin", [(4, 0, 0), (16, 1, 0), (8, 2, 0), (1, 3, 0), (8, 0, 40), (8, 0, 255),
                                                       (8, 0, 1000), (8, 4, 0), (8, 8, 0), (2, 9, 5)])
def test_tile_schedules_and_cu_margin_do_not_change_a_bit(raster_rows, flags, margin):
    """Launch tuning (raster group height, whole tail tiles, no half tiles) and sm_margin move tiles between
    workgroups; every output bit must stay what the default schedule gives."""
    from flux_amd import capi
    rng = np.random.default_rng(5)
    g = torch.Generator().manual_seed(5)
    experts, rows, n, kk = 6, 5000, 768, 512
    cnt = rng.multinomial(rows, [0.4, 0.02, 0.0, 0.28, 0.2, 0.1]).astype(np.int32)
    a = torch.randn(rows, kk, generator=g).to(torch.bfloat16).cuda()
    w = (torch.randn(experts, n, kk, generator=g) * 0.05).to(torch.bfloat16).cuda()
    sp = torch.from_numpy(cnt).cuda()
    base = capi.grouped_gemm(a, w, sp)
    close(base, layers.grouped_gemm_fp32(a.cpu(), w.cpu(), cnt))
    got = capi.grouped_gemm(a, w, sp, cu_margin=margin, raster_rows=raster_rows, sched_flags=flags)
    assert torch.equal(got, base)


def test_sm_margin_through_the_ops(c1):
    wl = c1
    t, k, e, h, f = wl.tokens, wl.topk, wl.experts, wl.hidden, wl.ffn
    x, w1 = wl.tensors["x"].cuda(), wl.tensors["w1"].cuda()
    op0 = flux_amd.GemmGroupedV3AGScatter(flux_amd.DistEnvTPWithEP(None, 1, None),
                                          flux_amd.MoeArguments(t, h, f, e, k, torch.bfloat16))
    sp, si = torch.from_numpy(wl.splits).cuda(), torch.from_numpy(wl.scatter_index).cuda()
    assert torch.equal(op0.forward(x, w1, sp, si, sm_margin=28), op0.forward(x, w1, sp, si))
    with pytest.raises(RuntimeError, match="sm_margin"):
        op0.forward(x, w1, sp, si, sm_margin=-1)


def test_blockscale_gemm_op_dense_and_grouped():
    """BlockScaleGemm.forward / forward_grouped / forward_multistream / reference (src/pybind/gemm_only.cc:77-160) fed by the Quantization op, the way
    test/python/gemm_only/test_blockwise_scale_gemm_only.py drives them: both scale layouts of forward_grouped."""
    g = torch.Generator().manual_seed(12)
    experts, n, k = 3, 384, 512
    split = np.array([200, 0, 313], dtype=np.int32)
    m = int(split.sum())
    x = torch.randn(m, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(experts, n, k, generator=g) * 0.05).to(torch.bfloat16)
    q = flux_amd.Quantization(torch.bfloat16, torch.float8_e4m3fn)
    qx, sx, _, _ = q.quantize_vector_blockwise(x.cuda(), return_tranpose=False)          # [ceil(M/128), K/128, 128]
    qw, sw, _, _ = q.batch_quantize_square_blockwise(w.cuda(), return_tranpose=False)    # [E, N/128, K/128]
    op = flux_amd.BlockScaleGemm(torch.float8_e4m3fn, torch.float8_e4m3fn, torch.bfloat16)
    sa = sx.cpu().permute(0, 2, 1).reshape(-1, k // 128)[:m]
    ref = layers.fp8_blockscale_grouped_gemm_fp32(qx.cpu(), sa, qw.cpu(), sw.cpu(), split)
    out = op.forward_grouped(qx, torch.from_numpy(split), qw, input_scale=sx, weight_scale=sw)
    assert out.dtype == torch.bfloat16
    assert torch.allclose(out.float().cpu(), ref, rtol=1e-2, atol=1e-2 * float(ref.abs().max()))
    # the reference's operand layouts: flat per-expert [K/128, M_e] and [K/128, N/128]
    flat_a = layers.a_scale_to_expert_k_m(sa, split).cuda()
    flat_b = sw.transpose(1, 2).contiguous().reshape(-1)
    out2 = op.forward_grouped(qx, torch.from_numpy(split), qw, input_scale=flat_a, weight_scale=flat_b)
    assert torch.equal(out2, out)
    # dense
    d = op.forward(qx, qw[0], input_scale=sx, weight_scale=sw[0].contiguous())
    refd = layers.fp8_blockscale_grouped_gemm_fp32(qx.cpu(), sa, qw.cpu()[:1], sw.cpu()[:1], np.array([m], dtype=np.int32))
    assert torch.allclose(d.float().cpu(), refd, rtol=1e-2, atol=1e-2 * float(refd.abs().max()))
    # the multi-stream form's arguments (blockscale_gemm.cc:376-486): input_scale [M, K/128] as the transposed view of a
    # [K/128, M] tensor, weight_scale [E, N/128, K/128]; same launch, same bits
    sa_t = sa.t().contiguous().cuda().t()
    assert sa_t.shape == (m, k // 128) and not sa_t.is_contiguous()
    out3 = op.forward_multistream(qx, torch.from_numpy(split), qw, input_scale=sa_t, weight_scale=sw)
    assert torch.equal(out3, out)
    # the reference's second implementation and its tuning entry point: one kernel here
    assert torch.equal(op.reference(qx, qw[0], input_scale=sx, weight_scale=sw[0].contiguous()), d)
    assert torch.equal(op.profiling(qx, qw[0], input_scale=sx, weight_scale=sw[0].contiguous()), d)
    # is_groupwise_b: one weight scale per column and 128 of K, [N/128, K/128, 128] (test_blockwise_scale_gemm_only.py:209,
    # 237-240); the oracle is the same dequantise-matmul with the scale taken per column
    gq = torch.Generator().manual_seed(13)
    swc = (torch.rand(n // 128, k // 128, 128, generator=gq) + 0.5) * float(sw[0].mean())
    dq = op.reference(qx, qw[0], input_scale=sx, weight_scale=swc.cuda(), is_groupwise_b=True)
    wq = qw[0].cpu().float().reshape(n // 128, 128, k // 128, 128) * swc.permute(0, 2, 1)[:, :, :, None]
    aq = qx.cpu().float().reshape(m, k // 128, 128) * sa[:, :, None]
    refq = aq.reshape(m, k) @ wq.reshape(n, k).t()
    assert torch.allclose(dq.float().cpu(), refq, rtol=1e-2, atol=1e-2 * float(refq.abs().max()))
    with pytest.raises(RuntimeError, match="per-column weight_scale"):
        op.reference(qx, qw[0], input_scale=sx, weight_scale=sw[0].contiguous(), is_groupwise_b=True)
    with pytest.raises(RuntimeError, match="bias"):
        op.forward(qx, qw[0], bias=torch.zeros(1, device="cuda"), input_scale=sx, weight_scale=sw[0].contiguous())
    with pytest.raises(RuntimeError, match="cpu"):
        op.forward_grouped(qx, torch.from_numpy(split).cuda(), qw, input_scale=sx, weight_scale=sw)
    # scales of the right size in another arrangement are rejected instead of being read in the wrong layout
    assert n // 128 != k // 128
    with pytest.raises(RuntimeError, match="weight_scale must be"):
        op.forward_grouped(qx, torch.from_numpy(split), qw, input_scale=sx, weight_scale=sw.transpose(1, 2).contiguous())
    with pytest.raises(RuntimeError, match="input_scale must be"):
        op.forward_grouped(qx, torch.from_numpy(split), qw, input_scale=sa.contiguous().cuda(), weight_scale=sw)
    with pytest.raises(RuntimeError, match="input_scale must be"):
        op.forward(qx, qw[0], input_scale=sx.reshape(-1), weight_scale=sw[0].contiguous())


def test_layer1_op_with_the_fused_epilogue_reduce(c1, monkeypatch):
    """FLUX_AMD_LAYER1_REDUCE=fused: the layer1 op reduces in the GEMM's epilogue; same bound, and at top-2 the same
    bits as the default two-pass form."""
    wl = c1
    t, k, e, h = wl.tokens, wl.topk, wl.experts, wl.hidden
    act, w2 = wl.tensors["act"].cuda(), wl.tensors["w2"].cuda()
    splits_cpu = torch.from_numpy(wl.splits)
    idx = torch.from_numpy(wl.scatter_index.reshape(-1)).cuda()
    ovs = wl.row_weight.cuda()
    base = flux_amd.GemmGroupedV3GatherRS(e, t * k, h, k, 0, 1, 1, 1).forward_gather_rs(act, w2, splits_cpu, idx,
                                                                                      output_vec_scale=ovs)
    monkeypatch.setenv("FLUX_AMD_LAYER1_REDUCE", "fused")
    op = flux_amd.GemmGroupedV3GatherRS(e, t * k, h, k, 0, 1, 1, 1)
    monkeypatch.delenv("FLUX_AMD_LAYER1_REDUCE")
    s_in, s_w = torch.tensor([0.75]), torch.rand(e) + 0.5
    out = op.forward_gather_rs(act, w2, splits_cpu, idx, output_vec_scale=ovs)
    ref = layers.layer1_fp32(wl.tensors["act"], wl.tensors["w2"], wl.splits, wl.scatter_index.reshape(-1), k,
                             output_vec_scale=wl.row_weight)
    close(out, ref)
    assert torch.equal(out, base)
    outs = op.forward_gather_rs(act, w2, splits_cpu, idx, input_scale=s_in.cuda(), weight_scale=s_w.cuda(),
                                output_vec_scale=ovs)
    close(outs, layers.layer1_fp32(wl.tensors["act"], wl.tensors["w2"], wl.splits, wl.scatter_index.reshape(-1), k,
                                   s_in, s_w, wl.row_weight))
    monkeypatch.setenv("FLUX_AMD_LAYER1_REDUCE", "sideways")
    with pytest.raises(RuntimeError, match="FLUX_AMD_LAYER1_REDUCE"):
        flux_amd.GemmGroupedV3GatherRS(e, t * k, h, k, 0, 1, 1, 1)


def test_layer1_intermediate_dtype_is_a_constructor_option(c1):
    """inter_dtype (after the reference's ten constructor arguments): fp32 by default, the 16-bit output type on
    request — the reference's own data flow, checked at the reference's own bound for it (2e-2 / 2e-2,
    test/python/moe_gather_rs/test_moe_gather_rs.py:397-411)."""
    wl = c1
    t, k, e, h, f = wl.tokens, wl.topk, wl.experts, wl.hidden, wl.ffn
    y = layers.layer0_fp32(wl.tensors["x"], wl.tensors["w1"], wl.splits, wl.gather_index).to(torch.bfloat16).cuda()
    w2 = wl.tensors["w2"].cuda()
    idx = torch.from_numpy(wl.scatter_index.reshape(-1)).cuda()
    ovs = wl.row_weight.cuda()
    ref = layers.layer1_fp32(y.cpu(), wl.tensors["w2"], wl.splits, wl.scatter_index.reshape(-1), k, output_vec_scale=wl.row_weight)
    outs = {}
    for name, dt in (("default", None), ("fp32", torch.float32), ("bf16", torch.bfloat16)):
        op = flux_amd.GemmGroupedV3GatherRS(e, t * k, h, k, 0, 1, 1, 1, inter_dtype=dt)
        outs[name] = op.forward_gather_rs(y, w2, torch.from_numpy(wl.splits), idx, output_vec_scale=ovs)
    assert torch.equal(outs["default"], outs["fp32"])
    close(outs["fp32"], ref)
    got = outs["bf16"].float().cpu()
    assert torch.allclose(got, ref, rtol=2e-2, atol=2e-2), float((got - ref).abs().max())
    assert not torch.equal(outs["bf16"], outs["fp32"])  # the terms really were rounded before the sum
    with pytest.raises(RuntimeError, match="inter_dtype"):
        flux_amd.GemmGroupedV3GatherRS(e, t * k, h, k, 0, 1, 1, 1, inter_dtype=torch.int32)
