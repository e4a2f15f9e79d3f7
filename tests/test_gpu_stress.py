"""Stress in the spirit of the reference's test/python/stress/stress_moe_{ag_scatter,gather_rs}.py: random token
counts, expert counts and skewed routing per iteration through the whole step (route sort -> layer0 -> layer1
-> reduce), each iteration checked against fp32 torch matmuls of the same inputs on the GPU (the CPU oracle pins
the kernels in the other test files; here the point is many ragged shapes, empty experts and tail tiles)."""
import numpy as np
import pytest
import torch

from oracle import routing

pytestmark = pytest.mark.gpu


def reference_step(x, w1, w2, choosed, topk_w, experts):
    t, k = choosed.shape
    out = torch.zeros(t, w2.shape[1], dtype=torch.float32, device=x.device)
    for e in range(experts):
        tok, slot = torch.nonzero(choosed == e, as_tuple=True)
        if tok.numel() == 0:
            continue
        y = (x[tok].float() @ w1[e].float().t()).to(torch.bfloat16)          # layer0 rounds to bf16
        z = y.float() @ w2[e].float().t()
        out.index_add_(0, tok, z * topk_w[tok, slot][:, None])
    return out


@pytest.mark.parametrize("seed", range(12))
def test_random_ragged_steps(seed):
    from flux_amd import capi
    rng = np.random.default_rng(1000 + seed)
    experts = int(rng.choice([1, 2, 3, 8, 17, 64]))
    topk = int(rng.integers(1, min(experts, 8) + 1))
    tokens = int(rng.integers(1, 3000))
    hidden = int(rng.choice([64, 256, 320, 1024]))
    ffn = int(rng.choice([128, 264, 384, 1408]))
    skew = float(rng.choice([0.0, 1.2, 3.0]))
    print(f"[case] stress seed={seed} T={tokens} k={topk} E={experts} H={hidden} F={ffn} skew={skew}", flush=True)
    g = torch.Generator(device="cuda").manual_seed(seed)
    p = torch.arange(1, experts + 1, dtype=torch.float32, device="cuda") ** -skew
    if experts > 2:
        p[int(rng.integers(0, experts))] = 0.0 if experts - 1 >= topk else p[0]   # an expert nobody picks
    if int((p > 0).sum()) < topk:
        p = torch.ones_like(p)
    choosed = torch.multinomial(p.repeat(tokens, 1), topk, replacement=False, generator=g).to(torch.int32)
    topk_w = torch.softmax(torch.randn(tokens, topk, generator=g, device="cuda"), dim=-1)
    x = torch.randn(tokens, hidden, generator=g, device="cuda").to(torch.bfloat16)
    w1 = (torch.randn(experts, ffn, hidden, generator=g, device="cuda") * hidden ** -0.5).to(torch.bfloat16)
    w2 = (torch.randn(experts, hidden, ffn, generator=g, device="cuda") * ffn ** -0.5).to(torch.bfloat16)

    splits, offsets, scatter, gather, tki = capi.route_sort(choosed, experts)
    c = choosed.cpu().numpy()
    assert np.array_equal(splits.cpu().numpy(), routing.splits(c, experts))
    assert np.array_equal(scatter.cpu().numpy(), routing.scatter_index_stable(c, experts))
    row_w = torch.empty(tokens * topk, dtype=torch.float32, device="cuda")
    row_w[scatter.reshape(-1).long()] = topk_w.reshape(-1)
    y = capi.grouped_gemm(x, w1, splits, gather_a=gather)
    z = capi.grouped_gemm(y, w2, splits, row_scale=row_w, out_dtype=torch.float32)
    out = capi.topk_gather_reduce(z, scatter.reshape(-1), topk)
    ref = reference_step(x, w1, w2, choosed, topk_w, experts)
    got = out.float()
    bad = (got - ref).abs() > 1e-2 + 1e-2 * ref.abs()
    assert not bool(bad.any()), f"{int(bad.sum())} of {bad.numel()} outside tolerance, max {float((got - ref).abs().max())}"


@pytest.mark.parametrize("seed", range(10))
@pytest.mark.parametrize("dtype", ["bf16", "fp8"])
def test_random_ragged_gemms_all_tile_shapes(dtype, seed):
    """One grouped GEMM per case over random splits (empty and tiny experts included), N that ends in a narrow
    column tile or not, K from one k-step to fifty, and enough rows that some cases run more tiles than CUs and
    cut their last round into pieces; per-row and per-column scales in the epilogue.  Reference: fp32 matmuls of
    the same values on the GPU."""
    from flux_amd import capi
    rng = np.random.default_rng(5000 + seed)
    experts = int(rng.choice([1, 3, 8, 32]))
    rows = int(rng.choice([37, 900, 5000, 20000, 40000]))
    n = int(rng.choice([128, 264, 384, 1024, 2048]))
    kbytes = int(rng.choice([64, 640, 1280, 2048, 3200]))
    k = kbytes if dtype == "fp8" else kbytes // 2
    p = rng.random(experts) ** 3 + 1e-3
    if experts > 2:
        p[int(rng.integers(0, experts))] = 0.0
    split = rng.multinomial(rows, p / p.sum()).astype(np.int32)
    print(f"[case] stress gemm {dtype} seed={seed} E={experts} rows={rows} N={n} K={k} split[:8]={split[:8]}", flush=True)
    g = torch.Generator(device="cuda").manual_seed(seed)
    a = torch.randn(rows, k, generator=g, device="cuda")
    w = torch.randn(experts, n, k, generator=g, device="cuda") * (1.0 if dtype == "fp8" else k ** -0.5)
    a = a.to(torch.float8_e4m3fn if dtype == "fp8" else torch.bfloat16)
    w = w.to(torch.float8_e4m3fn if dtype == "fp8" else torch.bfloat16)
    rs = torch.rand(rows, generator=g, device="cuda") + 0.5
    cs = (torch.rand(experts, n, generator=g, device="cuda") + 0.5) * (k ** -0.5 if dtype == "fp8" else 1.0)
    # odd seeds: A is gathered through a permutation and D scattered through another one
    gather = scatter = None
    src = a
    if seed % 2:
        gather = torch.randperm(rows, generator=g, device="cuda").to(torch.int32)
        scatter = torch.randperm(rows, generator=g, device="cuda").to(torch.int32)
        src = torch.empty_like(a)
        src.view(torch.uint8 if dtype == "fp8" else torch.int16)[gather.long()] = \
            a.view(torch.uint8 if dtype == "fp8" else torch.int16)          # src[gather[r]] = a[r]
    out = capi.grouped_gemm(src, w, torch.from_numpy(split).cuda(), row_scale=rs, col_scale=cs, gather_a=gather,
                            scatter_d=scatter).float()
    if scatter is not None:
        out = out[scatter.long()]                                           # back to sorted-row order
    ref = torch.zeros(rows, n, dtype=torch.float32, device="cuda")
    off = 0
    for e, cnt in enumerate(split):
        cnt = int(cnt)
        if cnt:
            ref[off:off + cnt] = (a[off:off + cnt].float() @ w[e].float().t()) * rs[off:off + cnt, None] * cs[e][None, :]
        off += cnt
    bad = (out - ref).abs() > 1e-2 + 1e-2 * ref.abs()
    assert not bool(bad.any()), f"{int(bad.sum())} of {bad.numel()} outside tolerance, max {float((out - ref).abs().max())}"
