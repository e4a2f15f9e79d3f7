"""Pins oracle.layers against brute-force loops, float64 library matmuls and the reference tests' closed-form data."""
import numpy as np
import pytest
import torch

from oracle import configs, layers, routing


def tiny_case(seed=0, tokens=12, topk=3, experts=4, h=16, f=24):
    g = torch.Generator().manual_seed(seed)
    choosed = torch.stack([torch.randperm(experts, generator=g)[:topk] for _ in range(tokens)]).to(torch.int32)
    x = torch.randn(tokens, h, generator=g).to(torch.bfloat16)
    w1 = (torch.randn(experts, f, h, generator=g) * 0.1).to(torch.bfloat16)
    w2 = (torch.randn(experts, h, f, generator=g) * 0.1).to(torch.bfloat16)
    c = choosed.numpy()
    split = routing.splits(c, experts)
    si = routing.scatter_index_stable(c, experts)
    gi, ti = routing.gather_index(si, topk)
    return dict(tokens=tokens, topk=topk, experts=experts, h=h, f=f, choosed=c, x=x, w1=w1, w2=w2, split=split,
                si=si, gi=gi, ti=ti, g=g)


def test_layer0_against_python_loops_and_float64():
    c = tiny_case()
    out = layers.layer0_fp32(c["x"], c["w1"], c["split"], c["gi"])
    eor = routing.expert_of_row(c["split"])
    x64, w64 = c["x"].double().numpy(), c["w1"].double().numpy()
    ref = np.zeros((len(eor), c["f"]))
    for r in range(len(eor)):
        for n in range(c["f"]):
            ref[r, n] = sum(x64[c["gi"][r], k] * w64[eor[r], n, k] for k in range(c["h"]))
    assert np.allclose(out.numpy(), ref, rtol=1e-5, atol=1e-6)
    # a transposed weight or a swapped gather would fail these:
    assert not np.allclose(out.numpy(), ref[::-1], rtol=1e-2, atol=1e-3)


def test_layer0_scale_and_rounding_forms_agree_within_bf16():
    c = tiny_case(1)
    alpha = torch.tensor([0.5, 2.0, 1.5, 0.25])
    a = layers.layer0_fp32(c["x"], c["w1"], c["split"], c["gi"], alpha)
    b = layers.layer0_torch(c["x"], c["w1"], c["split"], c["gi"], alpha).float()
    assert torch.allclose(a, b, rtol=2e-2, atol=1e-2)
    un = layers.layer0_fp32(c["x"], c["w1"], c["split"], c["gi"])
    eor = torch.as_tensor(routing.expert_of_row(c["split"]), dtype=torch.long)
    assert torch.allclose(a, un * alpha[eor][:, None], rtol=1e-6, atol=1e-7)


def test_single_expert_reduces_to_dense_matmul():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(40, 32, generator=g).to(torch.bfloat16)
    w = torch.randn(1, 48, 32, generator=g).to(torch.bfloat16)
    out = layers.grouped_gemm_fp32(x, w, np.array([40], dtype=np.int32))
    assert torch.allclose(out, x.float() @ w[0].float().t(), rtol=1e-6, atol=1e-6)
    # empty experts leave rows untouched and change nothing else
    w3 = torch.cat([w, w, w])
    out3 = layers.grouped_gemm_fp32(x, w3, np.array([0, 40, 0], dtype=np.int32))
    assert torch.equal(out, out3)


def test_gather_reduce_against_loop_form():
    """weights == 1: the loop of test/python/util/test_scatter_only.py:79-96."""
    c = tiny_case(2)
    m = c["tokens"] * c["topk"]
    inter = torch.randn(m, 8, generator=c["g"]).to(torch.bfloat16)
    idx = c["si"].reshape(-1)
    out = layers.topk_gather_reduce_fp32(inter, idx, c["topk"])
    ref = torch.zeros(c["tokens"], 8)
    for i in range(m):
        ref[i // c["topk"]] += inter[int(idx[i])].float()
    assert torch.allclose(out, ref, rtol=1e-6, atol=1e-6)
    w = torch.rand(m, generator=c["g"])
    outw = layers.topk_gather_reduce_fp32([inter, inter], idx, c["topk"], w, scale=0.5)
    refw = torch.zeros(c["tokens"], 8)
    for i in range(m):
        refw[i // c["topk"]] += 2 * 0.5 * w[int(idx[i])] * inter[int(idx[i])].float()
    assert torch.allclose(outw, refw, rtol=1e-5, atol=1e-6)
    # identity routing with k = 1 is a copy
    ident = layers.topk_gather_reduce_fp32(inter, np.arange(m), 1)
    assert torch.equal(ident, inter.float())
    # dropped rows (index -1) contribute nothing
    idx2 = idx.copy()
    idx2[0] = -1
    out2 = layers.topk_gather_reduce_fp32(inter, idx2, c["topk"])
    assert torch.allclose(out2[0], out[0] - inter[int(idx[0])].float(), atol=1e-6)


def test_layer1_forms_agree():
    c = tiny_case(4)
    m = c["tokens"] * c["topk"]
    act = torch.randn(m, c["f"], generator=c["g"]).to(torch.bfloat16)
    w_row = torch.rand(m, generator=c["g"])
    s_in = torch.tensor([0.75])
    s_w = torch.tensor([1.0, 0.5, 2.0, 1.25])
    a = layers.layer1_fp32(act, c["w2"], c["split"], c["si"].reshape(-1), c["topk"], s_in, s_w, w_row)
    b = layers.layer1_torch(act, c["w2"], c["split"], c["gi"], c["ti"], c["topk"], s_in, s_w, w_row).float()
    assert torch.allclose(a, b, rtol=2e-2, atol=2e-2)
    # brute force
    eor = routing.expert_of_row(c["split"])
    ref = torch.zeros(c["tokens"], c["h"], dtype=torch.float64)
    for i in range(m):
        r = int(c["si"].reshape(-1)[i])
        ref[i // c["topk"]] += float(w_row[r]) * 0.75 * float(s_w[eor[r]]) * (act[r].double() @ c["w2"][eor[r]].double().t())
    assert torch.allclose(a.double(), ref, rtol=1e-5, atol=1e-6)


def test_layer1_torch_rounds_after_the_scalar_scale():
    """scale_v * torch.matmul(...) of the reference (python/flux/testing/moe_gather_rs_utils.py:89) is a python
    float times a bf16 tensor, i.e. bf16: the scaled product is rounded before output_vec_scale is applied.
    Hand-computed case that tells the two forms apart: y = 1.0078125 (bf16), scale_v = 1 + 2^-8, weight 0.998:
      three roundings: bf16(1.0117797...) = 1.015625 (above the midpoint 1.01171875), times 0.998 = 1.01359 -> 1.015625
      without the middle rounding: 1.0117797 * 0.998 = 1.009756 -> 1.0078125."""
    act = torch.tensor([[1.0]], dtype=torch.bfloat16)
    w = torch.tensor([[[1.0078125]]], dtype=torch.bfloat16)
    split = np.array([1], dtype=np.int32)
    gi, ti = np.array([0]), np.array([0])
    out = layers.layer1_torch(act, w, split, gi, ti, 1, None, torch.tensor([1.00390625]), torch.tensor([0.998]))
    assert out.dtype == torch.bfloat16 and float(out[0, 0]) == 1.015625
    assert float(torch.tensor(1.0078125 * 1.00390625 * 0.998).to(torch.bfloat16)) == 1.0078125  # the two-rounding value


def test_reference_debug_closed_form():
    """The --debug data of test/python/moe_gather_rs/test_moe_gather_rs.py:502-518: x[:,0] = (i+1) % M, rest 0,
    W = 1, output_vec_scale = 2  =>  every output column of token t equals 2 * sum_j x[row_j, 0]."""
    tokens, topk, experts, k, n = 16, 2, 4, 8, 8
    m = tokens * topk
    choosed = np.stack([np.arange(topk) + (t % (experts - topk + 1)) for t in range(tokens)]).astype(np.int32)
    split = routing.splits(choosed, experts)
    si = routing.scatter_index_stable(choosed, experts)
    gi, ti = routing.gather_index(si, topk)
    act = torch.zeros(m, k, dtype=torch.bfloat16)
    act[:, 0] = ((torch.arange(m) + 1) % m).to(torch.bfloat16)
    w = torch.ones(experts, n, k, dtype=torch.bfloat16)
    ovs = torch.full((m,), 2.0)
    out = layers.layer1_fp32(act, w, split, si.reshape(-1), topk, None, None, ovs)
    expect = torch.stack([2.0 * sum(act[int(si[t, j]), 0].float() for j in range(topk)) for t in range(tokens)])
    assert torch.equal(out, expect[:, None].expand(tokens, n))
    out_t = layers.layer1_torch(act, w, split, gi, ti, topk, None, None, ovs).float()
    assert torch.equal(out_t, out)


def test_fp8_dequant_matmul_form():
    from oracle import quant
    g = torch.Generator().manual_seed(7)
    x = torch.randn(24, 64, generator=g).to(torch.bfloat16)
    w = (torch.randn(2, 16, 64, generator=g) * 0.02).to(torch.bfloat16)
    qx, sx = quant.quant_rows(x.view(torch.int16).numpy().view(np.uint16))
    qw, sw = quant.quant_rows(w.reshape(32, 64).view(torch.int16).numpy().view(np.uint16))
    tq = lambda a: torch.from_numpy(a.copy()).view(torch.float8_e4m3fn)
    split = np.array([10, 14], dtype=np.int32)
    out = layers.fp8_grouped_gemm_fp32(tq(qx), torch.from_numpy(sx), tq(qw).reshape(2, 16, 64),
                                       torch.from_numpy(sw).reshape(2, 16), split)
    ref = layers.grouped_gemm_fp32(x, w, split)
    err = (out - ref).norm() / ref.norm()
    # e4m3 keeps 4 significant bits: ~3-5 % relative error against the unquantised product is inherent
    # (the benchmark's 3e-2 bound is against the dequantise-matmul itself); a wrong scale index gives O(1).
    assert 0 < err < 8e-2


def test_blockscale_gemm_against_the_promotion_loop():
    """The dequantise-by-block oracle against the promotion form written out as loops (float64): for every output
    element, sum over K blocks of a_scale[r, kb] * w_scale[e, n // 128, kb] * (sum of the block's products).  A wrong
    block index, a transposed scale or a scale applied per element instead of per block fails."""
    g = torch.Generator().manual_seed(11)
    rows, n, k, experts = 5, 130, 256, 2
    split = np.array([2, 3], dtype=np.int32)
    qa = torch.randn(rows, k, generator=g).to(torch.float8_e4m3fn)
    qw = torch.randn(experts, n, k, generator=g).to(torch.float8_e4m3fn)
    sa = torch.rand(rows, k // 128, generator=g) + 0.5
    sw = torch.rand(experts, (n + 127) // 128, k // 128, generator=g) + 0.5
    out = layers.fp8_blockscale_grouped_gemm_fp32(qa, sa, qw, sw, split)
    eor = routing.expert_of_row(split)
    ref = torch.zeros(rows, n, dtype=torch.float64)
    for r in range(rows):
        e = int(eor[r])
        for col in range(n):
            for kb in range(k // 128):
                blk = slice(kb * 128, (kb + 1) * 128)
                part = float((qa[r, blk].double() * qw[e, col, blk].double()).sum())
                ref[r, col] += float(sa[r, kb]) * float(sw[e, col // 128, kb]) * part
    assert torch.allclose(out.double(), ref, rtol=1e-5, atol=1e-5)
    # layouts: the permuted 128-row form and the per-expert [K/128, M_e] form hold the same numbers
    p128 = layers.a_scale_to_block128(sa)
    assert tuple(p128.shape) == (1, 2, 128) and float(p128[0, 1, 3]) == float(sa[3, 1]) and float(p128[0, 0, 100]) == 0.0
    ekm = layers.a_scale_to_expert_k_m(sa, split)
    assert float(ekm[2 * 2 + 1 * 3 + 2]) == float(sa[4, 1])  # expert 1 starts at 2 rows * 2 blocks; block 1, its row 2
