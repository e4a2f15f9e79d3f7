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
