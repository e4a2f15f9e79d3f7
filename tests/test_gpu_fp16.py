"""GPU parity of the fp16 variants (the reference generates fp16 forms of both MoE ops:
src/generator/gen_moe_ag_scatter.cc:26-39, gen_moe_gather_rs.cc:25-45, and tests them with atol 1e-2 / rtol 1e-3 on
layer0, test/python/moe_ag_scatter/test_moe_ag.py:530-531, and 1e-2 / 1e-2 on layer1,
test/python/moe_gather_rs/test_moe_gather_rs.py:397-411).  fp16 operands, fp32 accumulation, fp16 (or fp32) output;
the oracle is the fp32 matmul of the fp16-valued operands."""
import numpy as np
import pytest
import torch

import flux_amd
from oracle import configs, layers, routing

pytestmark = pytest.mark.gpu
ATOL, RTOL = 1e-2, 1e-3


def close16(got, ref, what=""):
    got = got.float().cpu()
    bad = (got - ref).abs() > ATOL + RTOL * ref.abs()
    assert not bool(bad.any()), f"{what}: {int(bad.sum())} of {bad.numel()} outside tolerance, max err {float((got - ref).abs().max())}"


@pytest.mark.parametrize("experts,rows,n,k,seed", [(1, 256, 256, 64, 0), (4, 1000, 512, 256, 1), (8, 2048, 1024, 1024, 2),
                                                   (3, 700, 1408, 2048, 3), (5, 830, 328, 1184, 4), (2, 40, 50, 72, 5)])
def test_fp16_grouped_gemm_against_oracle(experts, rows, n, k, seed):
    from flux_amd import capi
    print(f"[case] grouped_gemm fp16 E={experts} rows={rows} N={n} K={k}", flush=True)
    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    p = rng.random(experts) + 0.05
    split = rng.multinomial(rows, p / p.sum()).astype(np.int32)
    a = torch.randn(rows, k, generator=g).to(torch.float16)
    w = (torch.randn(experts, n, k, generator=g) * 0.05).to(torch.float16)
    ref = layers.grouped_gemm_fp32(a, w, split)
    out, kind = capi.grouped_gemm(a.cuda(), w.cuda(), torch.from_numpy(split).cuda(), want_kind=True)
    assert out.dtype == torch.float16
    assert kind == (1 if (k % 8 == 0 and n % 4 == 0) else 0)
    close16(out, ref, "fp16 plain")
    out32 = capi.grouped_gemm(a.cuda(), w.cuda(), torch.from_numpy(split).cuda(), out_dtype=torch.float32)
    assert torch.allclose(out32.cpu(), ref, rtol=1e-4, atol=1e-3)
    # products of fp16 values differ from products of the same values rounded to bf16: the kernel must not run the bf16 MFMA
    wrong = layers.grouped_gemm_fp32(a.to(torch.bfloat16), w.to(torch.bfloat16), split)
    assert float((out32.cpu() - ref).abs().max()) < 0.1 * float((wrong - ref).abs().max())


def test_fp16_gather_scatter_scales_and_weight_groups():
    from flux_amd import capi
    rng = np.random.default_rng(31)
    g = torch.Generator().manual_seed(31)
    tokens, topk, experts, h, n = 300, 3, 6, 256, 520
    choosed = np.stack([rng.permutation(experts)[:topk] for _ in range(tokens)]).astype(np.int32)
    split = routing.splits(choosed, experts)
    si = routing.scatter_index_stable(choosed, experts)
    gi, _ = routing.gather_index(si, topk)
    m = tokens * topk
    x = torch.randn(tokens, h, generator=g).to(torch.float16)
    w = (torch.randn(experts, n, h, generator=g) * 0.05).to(torch.float16)
    alpha = torch.rand(experts, generator=g) + 0.5
    rs = torch.rand(m, generator=g) + 0.5
    cs = torch.rand(experts, n, generator=g) + 0.5
    perm = torch.randperm(m, generator=g).to(torch.int32)
    xs = x[torch.as_tensor(gi, dtype=torch.long)]
    ref = layers.grouped_gemm_fp32(xs, w, split, alpha=alpha, row_scale=rs, col_scale=cs, scalar=0.5)
    ref_scattered = torch.zeros_like(ref)
    ref_scattered[perm.long()] = ref
    out = capi.grouped_gemm(x.cuda(), w.cuda(), torch.from_numpy(split).cuda(), gather_a=torch.from_numpy(gi).cuda(),
                            scatter_d=perm.cuda(), alpha=alpha.cuda(), row_scale=rs.cuda(), col_scale=cs.cuda(), scalar_scale=0.5)
    close16(out, ref_scattered, "fp16 gather+scatter+scales")
    w2 = w.flip(0).contiguous()
    outs = capi.grouped_gemm_multi(x.cuda(), [w.cuda(), w2.cuda()], torch.from_numpy(split).cuda(), gather_a=torch.from_numpy(gi).cuda())
    close16(outs[0], layers.grouped_gemm_fp32(xs, w, split), "group 0")
    close16(outs[1], layers.grouped_gemm_fp32(xs, w2, split), "group 1")


@pytest.mark.parametrize("in_dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("topk,groups", [(2, 1), (6, 1), (3, 2)])
def test_fp16_gather_reduce(in_dtype, topk, groups):
    from flux_amd import capi
    g = torch.Generator().manual_seed(17 + topk)
    tokens, n = 200, 1024
    m = tokens * topk
    inter = [torch.randn(m, n, generator=g).to(in_dtype) for _ in range(groups)]
    idx = torch.randperm(m, generator=g).to(torch.int32)
    idx[5] = -1
    w = torch.rand(m, generator=g) + 0.5
    ref = layers.topk_gather_reduce_fp32(inter, idx.numpy(), topk, row_weight=w, scale=0.75)
    out = capi.topk_gather_reduce([t.cuda() for t in inter], idx.cuda(), topk, row_weight=w.cuda(), scale=0.75,
                                  out_dtype=torch.float16)
    assert out.dtype == torch.float16
    close16(out, ref, "fp16 gather-reduce")


def test_fp16_layer0_layer1_chain_through_the_ops():
    """The reference's call sequence (examples/moe_flux_only.py:112-131) with fp16 tensors: fp16 in gives fp16 out."""
    wl = configs.make_workload("C1")
    t, k, e, h, f = wl.tokens, wl.topk, wl.experts, wl.hidden, wl.ffn
    x, w1, w2 = (wl.tensors[n].to(torch.float16) for n in ("x", "w1", "w2"))
    splits_gpu = torch.from_numpy(wl.splits).cuda()
    scatter_index = torch.from_numpy(wl.scatter_index).cuda()
    op0 = flux_amd.GemmGroupedV3AGScatter(flux_amd.DistEnvTPWithEP(None, 1, None),
                                          flux_amd.MoeArguments(t, h, f, e, k, torch.float16))
    alpha = torch.rand(e) + 0.5
    y = op0.forward(x.cuda(), w1.cuda(), splits_gpu, scatter_index, output_scale=alpha.cuda())
    assert y.dtype == torch.float16 and tuple(y.shape) == (t * k, f)
    close16(y, layers.layer0_fp32(x, w1, wl.splits, wl.gather_index, alpha), "layer0 fp16")
    op1 = flux_amd.GemmGroupedV3GatherRS(e, t * k, h, k, 0, 1, 1, 1)
    out = op1.forward_gather_rs(y, w2.cuda(), torch.from_numpy(wl.splits), scatter_index.view(-1),
                                output_vec_scale=wl.row_weight.cuda())
    assert out.dtype == torch.float16 and tuple(out.shape) == (t, h)
    ref1 = layers.layer1_fp32(y.cpu(), w2, wl.splits, wl.scatter_index.reshape(-1), k, output_vec_scale=wl.row_weight)
    got = out.float().cpu()
    assert torch.allclose(got, ref1, rtol=1e-2, atol=1e-2), float((got - ref1).abs().max())
    # the fused epilogue reduce rounds to fp16 as well
    from flux_amd import capi
    fused = capi.grouped_gemm_topk_reduce(y, w2.cuda(), splits_gpu, torch.from_numpy(wl.gather_index).cuda(), t,
                                          row_scale=wl.row_weight.cuda())
    assert fused.dtype == torch.float16 and torch.equal(fused, out)
    # plain grouped GEMM op and the reduce op
    pg = flux_amd.GemmGroupedV3(w1.cuda(), e).forward(x.cuda()[torch.from_numpy(wl.gather_index).long().cuda()], torch.from_numpy(wl.splits))
    assert pg.dtype == torch.float16
    close16(pg, layers.layer0_fp32(x, w1, wl.splits, wl.gather_index), "GemmGroupedV3 fp16")
    red = flux_amd.topk_scatter_reduce([y], scatter_index, k)
    assert red.dtype == torch.float16
    with pytest.raises(RuntimeError, match="output dtype"):
        flux_amd.GemmGroupedV3AGScatter(flux_amd.DistEnvTPWithEP(None, 1, None),
                                        flux_amd.MoeArguments(t, h, f, e, k, torch.float16, torch.bfloat16))
