"""GPU parity, grouped GEMM (bf16 and fp8): bf16 outputs within rtol 1e-2 / atol 1e-2 of the fp32-accumulated
oracle; fp8 outputs within 3e-2 relative Frobenius error of the dequantise-matmul oracle."""
import numpy as np
import pytest
import torch

from oracle import configs, layers, quant, routing

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-2, 1e-2
FP8_FROB = 3e-2



@pytest.fixture(autouse=True, params=["half_line_fills", "whole_line_fills"])
def fill_form(request):
    """Every test of this module runs with both forms of the MFMA kernel's ring fills."""
    from flux_amd import capi
    capi.default_fill_form = capi.SCHED_HALF_LINE_FILLS if request.param == "half_line_fills" else capi.SCHED_WHOLE_LINE_FILLS
    yield request.param
    capi.default_fill_form = 0

def assert_close(got_bf16, ref_f32, what=""):
    got = got_bf16.float().cpu()
    bad = (got - ref_f32).abs() > ATOL + RTOL * ref_f32.abs()
    assert not bool(bad.any()), f"{what}: {int(bad.sum())} of {bad.numel()} outside tolerance, max err " \
                                f"{float((got - ref_f32).abs().max())}"


def random_splits(rng, experts, rows, empty=()):
    p = rng.random(experts) + 0.05
    for e in empty:
        p[e] = 0
    cnt = rng.multinomial(rows, p / p.sum())
    return cnt.astype(np.int32)


@pytest.mark.parametrize("experts,rows,n,k,seed,empty", [
    (1, 256, 256, 64, 0, ()), (1, 300, 264, 128, 1, ()), (4, 1000, 512, 256, 2, ()), (8, 2048, 1024, 1024, 3, (0, 5)),
    (3, 700, 1408, 2048, 4, (1,)), (16, 900, 256, 320, 5, (2, 3, 15)), (2, 17, 8, 32, 6, ()), (5, 1, 512, 64, 7, (0, 1, 2, 4)),
    (64, 6000, 384, 512, 8, ())])
def test_bf16_plain_against_oracle(experts, rows, n, k, seed, empty):
    from flux_amd import capi
    print(f"[case] grouped_gemm bf16 E={experts} rows={rows} N={n} K={k} empty={empty}", flush=True)
    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    split = random_splits(rng, experts, rows, empty)
    a = torch.randn(rows, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(experts, n, k, generator=g) * 0.05).to(torch.bfloat16)
    ref = layers.grouped_gemm_fp32(a, w, split)
    out = capi.grouped_gemm(a.cuda(), w.cuda(), torch.from_numpy(split).cuda())
    assert_close(out, ref, "plain")


def test_bf16_gather_scatter_and_scales():
    from flux_amd import capi
    rng = np.random.default_rng(21)
    g = torch.Generator().manual_seed(21)
    tokens, topk, experts, h, n = 300, 3, 6, 256, 520
    choosed = np.stack([rng.permutation(experts)[:topk] for _ in range(tokens)]).astype(np.int32)
    split = routing.splits(choosed, experts)
    si = routing.scatter_index_stable(choosed, experts)
    gi, _ = routing.gather_index(si, topk)
    m = tokens * topk
    x = torch.randn(tokens, h, generator=g).to(torch.bfloat16)
    w = (torch.randn(experts, n, h, generator=g) * 0.05).to(torch.bfloat16)
    alpha = torch.rand(experts, generator=g) + 0.5
    rs = torch.rand(m, generator=g) + 0.5
    cs = torch.rand(experts, n, generator=g) + 0.5
    sdev = torch.tensor([1.5])
    perm = torch.randperm(m, generator=g).to(torch.int32)
    xs = x[torch.as_tensor(gi, dtype=torch.long)]
    ref = layers.grouped_gemm_fp32(xs, w, split, alpha=alpha, row_scale=rs, col_scale=cs, scalar=0.5 * 1.5)
    ref_scattered = torch.zeros_like(ref)
    ref_scattered[perm.long()] = ref
    out = capi.grouped_gemm(x.cuda(), w.cuda(), torch.from_numpy(split).cuda(), gather_a=torch.from_numpy(gi).cuda(),
                            scatter_d=perm.cuda(), alpha=alpha.cuda(), row_scale=rs.cuda(), col_scale=cs.cuda(),
                            scalar_scale=0.5, scalar_scale_dev=sdev.cuda())
    assert_close(out, ref_scattered, "gather+scatter+scales")


@pytest.mark.parametrize("ngroups,experts,tokens,topk,h,n,seed,scaled", [
    (2, 4, 500, 2, 256, 520, 0, True),      # N not a whole number of macro tiles: the groups' column ranges are padded
    (3, 6, 300, 3, 320, 256, 1, False),
    (4, 2, 64, 1, 64, 8, 2, True),
    (2, 8, 4096, 2, 512, 1024, 3, True),    # 144 + tiles on 256 CUs: the last round is cut into pieces
    (2, 3, 40, 2, 72, 50, 4, True),         # K and N of the generic kernel
])
def test_bf16_multiple_weight_groups_one_launch(ngroups, experts, tokens, topk, h, n, seed, scaled):
    """forward_multiple_weights' kernel form: the same gathered rows times several weight tensors in one
    launch must equal one launch per weight tensor, and the oracle."""
    from flux_amd import capi
    print(f"[case] grouped_gemm_multi groups={ngroups} E={experts} T={tokens} k={topk} H={h} N={n}", flush=True)
    rng = np.random.default_rng(100 + seed)
    g = torch.Generator().manual_seed(100 + seed)
    choosed = np.stack([rng.permutation(experts)[:topk] for _ in range(tokens)]).astype(np.int32)
    split = routing.splits(choosed, experts)
    gi, _ = routing.gather_index(routing.scatter_index_stable(choosed, experts), topk)
    x = torch.randn(tokens, h, generator=g).to(torch.bfloat16)
    ws = [(torch.randn(experts, n, h, generator=g) * 0.05).to(torch.bfloat16) for _ in range(ngroups)]
    alphas = [torch.rand(experts, generator=g) + 0.5 if (scaled and i != 1) else None for i in range(ngroups)]
    xs = x[torch.as_tensor(gi, dtype=torch.long)]
    sp, gd, xd = torch.from_numpy(split).cuda(), torch.from_numpy(gi).cuda(), x.cuda()
    outs = capi.grouped_gemm_multi(xd, [w.cuda() for w in ws], sp, gather_a=gd,
                                   alphas=[None if al is None else al.cuda() for al in alphas] if scaled else None)
    assert len(outs) == ngroups
    for i in range(ngroups):
        ref = layers.grouped_gemm_fp32(xs, ws[i], split, alpha=alphas[i])
        assert_close(outs[i], ref, f"group {i}")
        single = capi.grouped_gemm(xd, ws[i].cuda(), sp, gather_a=gd, alpha=None if alphas[i] is None else alphas[i].cuda())
        assert torch.equal(outs[i], single), f"group {i}: one launch for all groups differs from a launch per group"


def test_multiple_weight_groups_argument_checks():
    from flux_amd import capi
    x = torch.zeros(8, 64, dtype=torch.bfloat16, device="cuda")
    w = torch.zeros(1, 8, 64, dtype=torch.bfloat16, device="cuda")
    sp = torch.tensor([8], dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match="ngroups"):
        capi.grouped_gemm_multi(x, [w] * 5, sp)


def test_bf16_generic_kernel_odd_shapes():
    """N not a multiple of 4, or rows of K that are not a multiple of 16 bytes, take the generic kernel."""
    from flux_amd import capi
    g = torch.Generator().manual_seed(31)
    split = np.array([13, 0, 20], dtype=np.int32)
    for n, k in ((50, 72), (52, 36)):
        a = torch.randn(33, k, generator=g).to(torch.bfloat16)
        w = (torch.randn(3, n, k, generator=g) * 0.1).to(torch.bfloat16)
        ref = layers.grouped_gemm_fp32(a, w, split)
        out, kind = capi.grouped_gemm(a.cuda(), w.cuda(), torch.from_numpy(split).cuda(), want_kind=True)
        assert kind == 0
        assert_close(out, ref, "generic")


@pytest.mark.parametrize("dtype,k", [("bf16", 8), ("bf16", 40), ("bf16", 72), ("bf16", 1000), ("bf16", 4104),
                                     ("bf16", 328), ("bf16", 456), ("bf16", 904),
                                     ("fp8", 16), ("fp8", 112), ("fp8", 1008), ("fp8", 4112), ("fp8", 1808)])
def test_k_not_a_multiple_of_the_k_step_runs_the_mfma_kernel(dtype, k):
    """Any K whose rows are a multiple of 16 bytes takes the MFMA kernel: the last, partial 64-byte step of K is
    completed with zeros inside the kernel.  Row counts cover full tiles, a 128-row tile and last-round pieces;
    the K values put the partial step into the prologue (K below four steps), into the pair-wise tail after
    unrolled trips, on an even and on an odd step, with 1, 2 and 3 valid chunks."""
    from flux_amd import capi
    print(f"[case] grouped_gemm {dtype} partial last k-step K={k}", flush=True)
    g = torch.Generator().manual_seed(k)
    split = np.array([300, 0, 129, 520, 77], dtype=np.int32)
    rows, n = int(split.sum()), 520
    if dtype == "bf16":
        a = torch.randn(rows, k, generator=g).to(torch.bfloat16)
        w = (torch.randn(len(split), n, k, generator=g) * 0.05).to(torch.bfloat16)
    else:
        a = torch.randn(rows, k, generator=g).to(torch.float8_e4m3fn)
        w = torch.randn(len(split), n, k, generator=g).to(torch.float8_e4m3fn)
    ref = layers.grouped_gemm_fp32(a.float(), w.float(), split)
    # a row's padding must be zeros: the bytes that follow a row in memory are the next row's values
    out32, kind = capi.grouped_gemm(a.cuda(), w.cuda(), torch.from_numpy(split).cuda(), out_dtype=torch.float32,
                                    want_kind=True)
    assert kind == 1, "the MFMA kernel must take this shape"
    assert torch.allclose(out32.cpu(), ref, rtol=1e-4, atol=1e-3 * max(1.0, k ** 0.5 if dtype == "fp8" else 1.0)), \
        float((out32.cpu() - ref).abs().max())
    if dtype == "bf16":
        out = capi.grouped_gemm(a.cuda(), w.cuda(), torch.from_numpy(split).cuda())
        assert_close(out, ref, f"K={k}")


def test_partial_k_step_with_gather_and_last_row_nan_guard():
    """The partial k-step together with a row gather: the last row of A ends the allocation's payload, and the
    rows are followed by NaN patterns that zero padding must never multiply in."""
    from flux_amd import capi
    g = torch.Generator().manual_seed(5)
    tokens, topk, experts, k, n = 200, 2, 3, 1000, 264
    rng = np.random.default_rng(5)
    choosed = np.stack([rng.permutation(experts)[:topk] for _ in range(tokens)]).astype(np.int32)
    split = routing.splits(choosed, experts)
    gi, _ = routing.gather_index(routing.scatter_index_stable(choosed, experts), topk)
    buf = torch.full((tokens + 1, k), float("nan"), dtype=torch.bfloat16)
    x = torch.randn(tokens, k, generator=g).to(torch.bfloat16)
    buf[:tokens] = x
    w = (torch.randn(experts, n, k, generator=g) * 0.05).to(torch.bfloat16)
    ref = layers.grouped_gemm_fp32(x[torch.as_tensor(gi, dtype=torch.long)], w, split)
    xd = buf.cuda()[:tokens]
    out, kind = capi.grouped_gemm(xd, w.cuda(), torch.from_numpy(split).cuda(), gather_a=torch.from_numpy(gi).cuda(),
                                  want_kind=True)
    assert kind == 1
    assert_close(out, ref, "gathered, K=1000")


def test_rows_beyond_splits_untouched():
    from flux_amd import capi
    g = torch.Generator().manual_seed(41)
    split = np.array([100, 50], dtype=np.int32)
    a = torch.randn(400, 64, generator=g).to(torch.bfloat16)
    w = (torch.randn(2, 256, 64, generator=g) * 0.1).to(torch.bfloat16)
    out = torch.full((400, 256), 7.0, dtype=torch.bfloat16, device="cuda")
    capi.grouped_gemm(a.cuda(), w.cuda(), torch.from_numpy(split).cuda(), out=out)
    ref = layers.grouped_gemm_fp32(a[:150], w, split)
    assert_close(out[:150], ref, "rows")
    assert bool((out[150:] == 7.0).all())


def test_single_expert_matches_dense_gemm():
    """E = 1 reduces to one dense GEMM: cross-check with torch.mm (hipBLASLt) on the GPU."""
    from flux_amd import capi
    gen = torch.Generator(device="cuda").manual_seed(51)
    a = torch.randn(1024, 2048, generator=gen, device="cuda").to(torch.bfloat16)
    w = (torch.randn(1, 768, 2048, generator=gen, device="cuda") * 0.02).to(torch.bfloat16)
    out = capi.grouped_gemm(a, w, torch.tensor([1024], dtype=torch.int32, device="cuda"))
    ref = (a.float() @ w[0].float().t()).cpu()
    assert_close(out, ref, "dense")


@pytest.mark.parametrize("k", [96, 160, 416, 448, 480, 544, 576, 608, 736, 768, 800, 864, 896, 928, 1312])
def test_bf16_k_loop_boundaries(k):
    """K lengths around the seams of the k loop: odd numbers of 64-byte k-steps (a phantom step on zeros), the
    hand-over from the unrolled trips of ten to the pair-wise tail (14 and 24 k-steps; 18 and 28 for the
    128x128 pieces with their deeper ring) and lengths on either side; rows chosen so that full tiles, a 128-row tile and last-round pieces all occur."""
    from flux_amd import capi
    print(f"[case] grouped_gemm bf16 k-loop seams K={k}", flush=True)
    g = torch.Generator().manual_seed(k)
    split = np.array([300, 0, 129, 520, 77], dtype=np.int32)
    rows, n = int(split.sum()), 520
    a = torch.randn(rows, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(len(split), n, k, generator=g) * 0.05).to(torch.bfloat16)
    ref = layers.grouped_gemm_fp32(a, w, split)
    out = capi.grouped_gemm(a.cuda(), w.cuda(), torch.from_numpy(split).cuda())
    assert_close(out, ref, f"K={k}")
    out32 = capi.grouped_gemm(a.cuda(), w.cuda(), torch.from_numpy(split).cuda(), out_dtype=torch.float32)
    assert torch.allclose(out32.cpu(), ref, rtol=1e-4, atol=1e-3), float((out32.cpu() - ref).abs().max())


@pytest.mark.parametrize("k", [192, 320, 832, 896, 960, 1088, 1152, 1216, 1472, 1536, 1600, 1728, 1792, 1856, 2624, 7168])
def test_fp8_k_loop_boundaries(k):
    """The same seams for the fp8 kernel (a k-step is 64 elements): every tile shape occurs (full tiles, 128-row
    tiles, the 8-column last tile as a 256x128 and a 128x128 tile), with K on either side of the hand-over from the
    unrolled trips to the pair-wise tail of each shape's ring, odd numbers of k-steps, and one long K."""
    from flux_amd import capi
    print(f"[case] grouped_gemm fp8 k-loop seams K={k}", flush=True)
    g = torch.Generator().manual_seed(k)
    split = np.array([300, 0, 129, 520, 77], dtype=np.int32)
    rows, n = int(split.sum()), 520
    a = torch.randn(rows, k, generator=g).to(torch.float8_e4m3fn)
    w = torch.randn(len(split), n, k, generator=g).to(torch.float8_e4m3fn)
    ref = layers.grouped_gemm_fp32(a.float(), w.float(), split)
    out32 = capi.grouped_gemm(a.cuda(), w.cuda(), torch.from_numpy(split).cuda(), out_dtype=torch.float32).cpu()
    # products of e4m3 values are exact in fp32; only the summation order differs
    assert torch.allclose(out32, ref, rtol=1e-4, atol=1e-3 * k ** 0.5), float((out32 - ref).abs().max())


def sampled_rows(split, per_expert, rng):
    off = routing.offsets(split)
    rows = []
    for e in range(len(split)):
        lo, hi = int(off[e]), int(off[e + 1])
        if hi == lo:
            continue
        pick = {lo, hi - 1, lo + (hi - lo) // 2}
        pick.update(int(v) for v in rng.integers(lo, hi, size=per_expert))
        rows.extend(sorted(pick))
    return np.array(rows, dtype=np.int64)


@pytest.mark.parametrize("name", ["C1", "C2", "C3", "C4"])
def test_benchmark_layer0_and_layer1(name):
    """The benchmark shapes at full size.  C1 is compared in full; the larger ones on a sample of sorted rows per
    expert (first, last, middle and random rows, all columns) computed by the oracle in fp32."""
    from flux_amd import capi
    wl = configs.make_workload(name, with_w2=(name != "C2"))
    print(f"[case] grouped_gemm {name} M={wl.rows} H={wl.hidden} F={wl.ffn} E={wl.experts}", flush=True)
    rng = np.random.default_rng(61)
    x, w1 = wl.tensors["x"], wl.tensors["w1"]
    split_d = torch.from_numpy(wl.splits).cuda()
    gi_d = torch.from_numpy(wl.gather_index).cuda()
    out0 = capi.grouped_gemm(x.cuda(), w1.cuda(), split_d, gather_a=gi_d)
    eor = routing.expert_of_row(wl.splits)
    rows = np.arange(wl.rows) if name == "C1" else sampled_rows(wl.splits, 6 if name == "C4" else 24, rng)
    for e in np.unique(eor[rows]):
        r = rows[eor[rows] == e]
        ref = x[torch.as_tensor(wl.gather_index[r], dtype=torch.long)].float() @ w1[int(e)].float().t()
        assert_close(out0[torch.as_tensor(r).cuda()], ref, f"{name} layer0 expert {e}")
    if name == "C2":
        return
    # layer1: grouped GEMM with the top-k weight in the epilogue, then the gather-reduce
    act, w2 = wl.tensors["act"], wl.tensors["w2"]
    z = capi.grouped_gemm(act.cuda(), w2.cuda(), split_d, row_scale=wl.row_weight.cuda())
    for e in np.unique(eor[rows]):
        r = rows[eor[rows] == e]
        ref = (act[torch.as_tensor(r)].float() @ w2[int(e)].float().t()) * wl.row_weight[torch.as_tensor(r)][:, None]
        assert_close(z[torch.as_tensor(r).cuda()], ref, f"{name} layer1 gemm expert {e}")
    idx_d = torch.from_numpy(wl.scatter_index.reshape(-1)).cuda()
    tok = rng.integers(0, wl.tokens, size=48)
    ref1 = torch.zeros(len(tok), wl.hidden)
    for i, t in enumerate(tok):
        for j in range(wl.topk):
            r = int(wl.scatter_index[t, j])
            ref1[i] += float(wl.row_weight[r]) * (act[r].float() @ w2[int(eor[r])].float().t())
    # (a) fp32 intermediate: one rounding in the whole layer -> the 1e-2 / 1e-2 bound against the fp32 oracle
    z32 = capi.grouped_gemm(act.cuda(), w2.cuda(), split_d, row_scale=wl.row_weight.cuda(), out_dtype=torch.float32)
    out32 = capi.topk_gather_reduce(z32, idx_d, wl.topk)
    assert_close(out32[torch.as_tensor(tok).cuda()], ref1, f"{name} layer1 output (fp32 intermediate)")
    # (b) bf16 intermediate, the reference's own data flow (inter_D is bf16:
    # src/moe_gather_rs/ths_op/gemm_grouped_v3_gather_rs.cc:620-631): every term carries a bf16 rounding, so
    # sums that cancel can miss 1e-2 absolute; the reference's own bound for this op is 2e-2 / 2e-2
    # (test/python/moe_gather_rs/test_moe_gather_rs.py:397-411).
    # With this benchmark's data (|z| reaches 8-16, where one bf16 step is 0.06) terms that cancel can miss a
    # flat 2e-2 by a rounding step, so the assertion is the a-priori bound of this data flow: every term and the
    # result are rounded once to bf16 (relative 2^-9 each), i.e. |err| <= 2^-8 * (sum_j w_j |z_j| + |ref|).  The flat
    # 2e-2 / 2e-2 must still hold for all but a vanishing fraction of the outputs.
    out1 = capi.topk_gather_reduce(z, idx_d, wl.topk)
    got = out1[torch.as_tensor(tok).cuda()].float().cpu()
    mag = torch.zeros(len(tok), wl.hidden)
    for i, t in enumerate(tok):
        for j in range(wl.topk):
            r = int(wl.scatter_index[t, j])
            mag[i] += (float(wl.row_weight[r]) * (act[r].float() @ w2[int(eor[r])].float().t())).abs()
    err = (got - ref1).abs()
    assert bool((err <= 2.0 ** -8 * (mag + ref1.abs()) + 1e-6).all()), float(err.max())
    flat_ok = err <= 2e-2 + 2e-2 * ref1.abs()
    assert float(flat_ok.float().mean()) >= 0.999, float(flat_ok.float().mean())


def quantise(t_bf16):
    bits = t_bf16.reshape(-1, t_bf16.shape[-1]).view(torch.int16).numpy().view(np.uint16)
    q, s = quant.quant_rows_c(bits)
    return torch.from_numpy(q).view(torch.float8_e4m3fn).reshape(t_bf16.shape), torch.from_numpy(s)


@pytest.mark.parametrize("experts,rows,n,k,seed", [(1, 256, 256, 64, 0), (4, 1000, 512, 256, 1), (8, 2000, 1024, 1024, 2),
                                                   (3, 300, 264, 2048, 3), (2, 40, 8, 100, 4), (3, 700, 264, 192, 5), (2, 300, 512, 960, 6), (4, 1100, 384, 1536, 7),
                                                   # 128x128 and 256x128 tiles (last rows of an expert, last columns of N) over
                                                   # 18 and more k-steps: the unrolled trips of the narrow tile shapes
                                                   (1, 100, 128, 2048, 8), (1, 100, 384, 1536, 9), (1, 256, 128, 1152, 10),
                                                   (2, 600, 640, 1280, 11)])
def test_fp8_against_dequant_matmul(experts, rows, n, k, seed):
    from flux_amd import capi
    print(f"[case] grouped_gemm fp8 E={experts} rows={rows} N={n} K={k}", flush=True)
    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    split = random_splits(rng, experts, rows)
    a = torch.randn(rows, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(experts, n, k, generator=g) * 0.02).to(torch.bfloat16)
    qa, sa = quantise(a)
    qw, sw = quantise(w)
    sw = sw.reshape(experts, n)
    tw = torch.rand(rows, generator=g) + 0.5
    ref = layers.fp8_grouped_gemm_fp32(qa, sa, qw, sw, split, row_weight=tw)
    out = capi.grouped_gemm(qa.cuda(), qw.cuda(), torch.from_numpy(split).cuda(), row_scale=(sa * tw).cuda(),
                            col_scale=sw.cuda())
    err = float((out.float().cpu() - ref).norm() / ref.norm())
    assert err < FP8_FROB, err
    assert err < 5e-3, err  # only accumulation order and the bf16 output rounding differ from the oracle


def test_fp8_benchmark_c5_layer1():
    """C5 at full size: quantise on the GPU, fp8 grouped GEMM with row x column scales and the top-8 weight in
    the epilogue, gather-reduce; sampled rows / tokens against the dequantise-matmul oracle."""
    from flux_amd import capi
    wl = configs.make_workload("C5")
    print(f"[case] grouped_gemm fp8 C5 M={wl.rows} K={wl.ffn} N={wl.hidden}", flush=True)
    rng = np.random.default_rng(71)
    act, w2 = wl.tensors["act"], wl.tensors["w2"]
    qa_d, sa_d = capi.quant_e4m3(act.cuda())
    qw_d, sw_d = capi.quant_e4m3(w2.reshape(-1, wl.ffn).cuda())
    qw_d = qw_d.reshape(wl.experts, wl.hidden, wl.ffn)
    sw_d = sw_d.reshape(wl.experts, wl.hidden)
    split_d = torch.from_numpy(wl.splits).cuda()
    z = capi.grouped_gemm(qa_d, qw_d, split_d, row_scale=sa_d * wl.row_weight.cuda(), col_scale=sw_d)
    out = capi.topk_gather_reduce(z, torch.from_numpy(wl.scatter_index.reshape(-1)).cuda(), wl.topk)
    eor = routing.expert_of_row(wl.splits)
    rows = sampled_rows(wl.splits, 8, rng)
    qa, sa, qw, sw = qa_d.cpu(), sa_d.cpu(), qw_d.cpu(), sw_d.cpu()
    num = den = 0.0
    for e in np.unique(eor[rows]):
        r = torch.as_tensor(rows[eor[rows] == e])
        ref = (qa[r].float() * sa[r][:, None]) @ (qw[int(e)].float() * sw[int(e)][:, None]).t() * wl.row_weight[r][:, None]
        num += float((z[r.cuda()].float().cpu() - ref).pow(2).sum())
        den += float(ref.pow(2).sum())
    assert (num / den) ** 0.5 < FP8_FROB
    tok = rng.integers(0, wl.tokens, size=16)
    ref1 = torch.zeros(len(tok), wl.hidden)
    for i, t in enumerate(tok):
        for j in range(wl.topk):
            r = int(wl.scatter_index[t, j])
            e = int(eor[r])
            ref1[i] += float(wl.row_weight[r]) * float(sa[r]) * ((qa[r].float() @ qw[e].float().t()) * sw[e])
    got = out[torch.as_tensor(tok).cuda()].float().cpu()
    assert float((got - ref1).norm() / ref1.norm()) < FP8_FROB


def test_fp8_benchmark_c5_layer0():
    """C5 layer0 at full size: tokens quantised per row on the GPU, weights per output channel, the row gather
    (C5's own gather_index, 32768 sorted rows from 4096 tokens) folded into the fp8 grouped GEMM, K = 7168,
    N = 2048; sampled rows against the dequantise-matmul oracle."""
    from flux_amd import capi
    wl = configs.make_workload("C5", with_w2=False)
    print(f"[case] grouped_gemm fp8 C5 layer0 M={wl.rows} K={wl.hidden} N={wl.ffn}", flush=True)
    rng = np.random.default_rng(72)
    x, w1 = wl.tensors["x"], wl.tensors["w1"]
    qx_d, sx_d = capi.quant_e4m3(x.cuda())
    qw_d, sw_d = capi.quant_e4m3(w1.reshape(-1, wl.hidden).cuda())
    qw_d = qw_d.reshape(wl.experts, wl.ffn, wl.hidden)
    sw_d = sw_d.reshape(wl.experts, wl.ffn)
    gi_d = torch.from_numpy(wl.gather_index).cuda()
    split_d = torch.from_numpy(wl.splits).cuda()
    # the per-row scale is indexed by sorted row: gather the per-token scales the same way as the rows
    rs_d = sx_d[gi_d.long()].contiguous()
    y, kind = capi.grouped_gemm(qx_d, qw_d, split_d, gather_a=gi_d, row_scale=rs_d, col_scale=sw_d, want_kind=True)
    assert kind == 1 and y.shape == (wl.rows, wl.ffn)
    eor = routing.expert_of_row(wl.splits)
    rows = sampled_rows(wl.splits, 8, rng)
    qx, sx, qw, sw = qx_d.cpu(), sx_d.cpu(), qw_d.cpu(), sw_d.cpu()
    num = den = 0.0
    for e in np.unique(eor[rows]):
        r = rows[eor[rows] == e]
        tok = torch.as_tensor(wl.gather_index[r], dtype=torch.long)
        ref = layers.fp8_grouped_gemm_fp32(qx[tok], sx[tok], qw[int(e):int(e) + 1], sw[int(e):int(e) + 1],
                                           np.array([len(r)], dtype=np.int32))
        got = y[torch.as_tensor(r).cuda()].float().cpu()
        num += float((got - ref).pow(2).sum())
        den += float(ref.pow(2).sum())
        assert torch.allclose(got, ref, rtol=2e-2, atol=2e-2 * float(ref.abs().max())), f"expert {e}"
    assert (num / den) ** 0.5 < FP8_FROB
    assert (num / den) ** 0.5 < 5e-3  # only accumulation order and the bf16 output rounding differ


def test_fp8_multiple_weight_groups_one_launch():
    from flux_amd import capi
    g = torch.Generator().manual_seed(77)
    experts, rows, n, k = 4, 1000, 384, 256
    split = random_splits(np.random.default_rng(77), experts, rows)
    a8 = torch.randn(rows, k, generator=g).to(torch.float8_e4m3fn)
    ws = [torch.randn(experts, n, k, generator=g).to(torch.float8_e4m3fn) for _ in range(2)]
    rs = torch.rand(rows, generator=g) + 0.5
    sp = torch.from_numpy(split).cuda()
    outs = capi.grouped_gemm_multi(a8.cuda(), [w.cuda() for w in ws], sp, row_scale=rs.cuda())
    for i in range(2):
        single = capi.grouped_gemm(a8.cuda(), ws[i].cuda(), sp, row_scale=rs.cuda())
        assert torch.equal(outs[i], single)
        ref = layers.grouped_gemm_fp32(a8.float(), ws[i].float(), split, row_scale=rs)
        err = (outs[i].float().cpu() - ref).norm() / ref.norm()
        assert float(err) < FP8_FROB


@pytest.mark.parametrize("dtype", ["bf16", "fp8"])
@pytest.mark.parametrize("row_tiles,what", [(17, "16 tiles past a full round: cut into 128x128 pieces"),
                                            (21, "80 tiles past a full round: cut into 256x128 pieces")])
def test_last_round_cut_into_pieces(dtype, row_tiles, what):
    """More tiles than CUs with a short last round (256 CUs, 16 column tiles): the schedule cuts the tiles of
    that round into pieces, which run the narrow tile shapes at every piece offset, here over 20 k-steps."""
    from flux_amd import capi
    print(f"[case] grouped_gemm {dtype} tail pieces, {row_tiles} row tiles x 16 column tiles: {what}", flush=True)
    g = torch.Generator().manual_seed(row_tiles)
    rows, n = 256 * row_tiles, 4096
    k = 640 if dtype == "bf16" else 1280          # 20 k-steps of 64 bytes
    split = np.array([rows - 700, 700], dtype=np.int32)
    if dtype == "bf16":
        a = torch.randn(rows, k, generator=g).to(torch.bfloat16)
        w = (torch.randn(2, n, k, generator=g) * 0.05).to(torch.bfloat16)
    else:
        a = torch.randn(rows, k, generator=g).to(torch.float8_e4m3fn)
        w = torch.randn(2, n, k, generator=g).to(torch.float8_e4m3fn)
    ref = layers.grouped_gemm_fp32(a.float(), w.float(), split)
    out = capi.grouped_gemm(a.cuda(), w.cuda(), torch.from_numpy(split).cuda()).float().cpu()
    if dtype == "bf16":
        assert_close(out, ref, what)
    else:
        assert float((out - ref).norm() / ref.norm()) < FP8_FROB
        assert torch.allclose(out, ref, rtol=1e-2, atol=1e-2 * float(ref.abs().max()))


@pytest.mark.parametrize("dtype", ["bf16", "fp8"])
@pytest.mark.parametrize("ksteps", [1, 2, 19, 35, 36, 37, 56, 57, 75])
def test_skinny_tail_pieces_same_bits_as_in_place(dtype, ksteps):
    """Experts whose last row tile holds 1 .. 64 rows: by default (when such tiles are few) that row tile runs behind all
    other tiles as 64 x 64 pieces on a ring of twenty 8 KiB stages.  Results must be what the oracle says and, bit for
    bit, what the schedule without skinny tails gives (FLUXMI_SCHED_NO_SKINNY_TAIL = 4; 8 forces them), over K
    lengths on both sides of the hand-over from the unrolled trips of twenty k-steps to the pair-wise tail (36
    k-steps), odd numbers of k-steps, with N that is not a multiple of 64, a gather, and every epilogue scale."""
    from flux_amd import capi
    elt = 2 if dtype == "bf16" else 1
    k = ksteps * 64 // elt
    print(f"[case] grouped_gemm {dtype} skinny tail pieces K={k} ({ksteps} k-steps)", flush=True)
    g = torch.Generator().manual_seed(100 + ksteps)
    split = np.array([300, 30, 257, 64, 65, 1, 0, 513, 256], dtype=np.int32)  # skinny: 300, 30, 257, 64, 1, 513
    rows, n = int(split.sum()), 328
    src_rows = rows + 37
    gi = torch.randint(0, src_rows, (rows,), generator=g, dtype=torch.int32)
    if dtype == "bf16":
        a = torch.randn(src_rows, k, generator=g).to(torch.bfloat16)
        w = (torch.randn(len(split), n, k, generator=g) * 0.05).to(torch.bfloat16)
    else:
        a = torch.randn(src_rows, k, generator=g).to(torch.float8_e4m3fn)
        w = (torch.randn(len(split), n, k, generator=g) * 0.25).to(torch.float8_e4m3fn)
    rs = torch.rand(rows, generator=g) + 0.5
    cs = torch.rand(len(split), n, generator=g) + 0.5
    ref = layers.grouped_gemm_fp32(a.float()[gi.long()], w.float(), split, row_scale=rs, col_scale=cs)
    sp = torch.from_numpy(split).cuda()
    kw = dict(gather_a=gi.cuda(), row_scale=rs.cuda(), col_scale=cs.cuda())
    for out_dtype in (torch.bfloat16, torch.float32):
        base = capi.grouped_gemm(a.cuda(), w.cuda(), sp, out_dtype=out_dtype, sched_flags=4, **kw)
        for flags in (0, 8):
            got = capi.grouped_gemm(a.cuda(), w.cuda(), sp, out_dtype=out_dtype, sched_flags=flags, **kw)
            assert torch.equal(got, base), f"sched_flags={flags} out={out_dtype}: bits differ from the in-place schedule"
        if out_dtype == torch.float32:
            assert torch.allclose(base.cpu(), ref, rtol=1e-4, atol=1e-3 * max(1.0, k ** 0.5 * (0.05 if dtype == "bf16" else 1.0)))
        elif dtype == "bf16":
            assert_close(base, ref, "skinny")
        else:
            assert float((base.float().cpu() - ref).norm() / ref.norm()) < 5e-3
    # plain (no gather, no scales: the unscaled epilogue), scattered rows, and two weight groups in one launch
    perm = torch.randperm(rows, generator=g).to(torch.int32).cuda()
    a2 = a[:rows].cuda()
    for kw2 in (dict(), dict(scatter_d=perm)):
        base = capi.grouped_gemm(a2, w.cuda(), sp, sched_flags=4, **kw2)
        got = capi.grouped_gemm(a2, w.cuda(), sp, sched_flags=8, **kw2)
        assert torch.equal(got, base)
    w2 = w.flip(0).contiguous().cuda()
    outs4 = capi.grouped_gemm_multi(a2, [w.cuda(), w2], sp, sched_flags=4)
    outs8 = capi.grouped_gemm_multi(a2, [w.cuda(), w2], sp, sched_flags=8)
    for o4, o8 in zip(outs4, outs8):
        assert torch.equal(o4, o8)


@pytest.mark.parametrize("dtype", ["bf16", "fp8"])
@pytest.mark.parametrize("k", [128, 1024, 1040, 4096])
def test_both_fill_forms_give_the_same_bits(dtype, k):
    """Half-line and whole-line ring fills walk K in the same order with the same MFMAs: ragged experts (whole,
    128-row, 64-row and partly filled tiles, pieces of the last round), a gather, a K with a partial last 128 bytes."""
    from flux_amd import capi
    rng = np.random.default_rng(k)
    rows = [300, 0, 257, 64, 1000, 129, 513, 40]
    m, n, tokens = sum(rows), 640, 700
    sp = torch.tensor(rows, dtype=torch.int32).cuda()
    gi = torch.from_numpy(rng.integers(0, tokens, m).astype(np.int32)).cuda()
    if dtype == "bf16":
        x = torch.from_numpy(rng.standard_normal((tokens, k), dtype=np.float32)).to(torch.bfloat16).cuda()
        w = torch.from_numpy(rng.standard_normal((len(rows), n, k), dtype=np.float32) * 0.05).to(torch.bfloat16).cuda()
    else:
        x = torch.from_numpy(rng.standard_normal((tokens, k), dtype=np.float32)).to(torch.float8_e4m3fn).cuda()
        w = torch.from_numpy(rng.standard_normal((len(rows), n, k), dtype=np.float32)).to(torch.float8_e4m3fn).cuda()
    for kw in (dict(gather_a=gi), dict(gather_a=gi, out_dtype=torch.float32)):
        half, kind = capi.grouped_gemm(x, w, sp, sched_flags=capi.SCHED_HALF_LINE_FILLS, want_kind=True, **kw)
        whole = capi.grouped_gemm(x, w, sp, sched_flags=capi.SCHED_WHOLE_LINE_FILLS, **kw)
        assert kind == 1
        assert torch.equal(half, whole), f"{dtype} k={k} {list(kw)}: the two fill forms differ"
    plain = x[gi.long()].contiguous()
    half = capi.grouped_gemm(plain, w, sp, sched_flags=capi.SCHED_HALF_LINE_FILLS)
    whole = capi.grouped_gemm(plain, w, sp, sched_flags=capi.SCHED_WHOLE_LINE_FILLS)
    assert torch.equal(half, whole)
    with pytest.raises(RuntimeError, match="at once"):
        capi.grouped_gemm(plain, w, sp, sched_flags=capi.SCHED_HALF_LINE_FILLS | capi.SCHED_WHOLE_LINE_FILLS)
