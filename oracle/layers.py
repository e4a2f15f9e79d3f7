"""Layer oracle: gathered grouped GEMM (layer0), grouped GEMM + top-k weighted gather-reduce (layer1).

PyTorch-CPU, fp32 accumulation on bf16-valued inputs.  Two flavours per layer:
  *_fp32   the fp32-accumulated target with no intermediate rounding (the tolerance reference)
  *_torch  the reference's own op order with its intermediate bf16 roundings
"""
import numpy as np
import torch

from . import routing


def _f32(t):
    return t.to(torch.float32)


def grouped_gemm_fp32(a_sorted, weights, split, alpha=None, row_scale=None, col_scale=None, scalar=1.0):
    """Per-expert x @ W[e].T on sorted rows, fp32 result
    (test/python/gemm_only/test_grouped_gemm_v3_only.py:55-66; weights are [E, N, K], K contiguous:
    src/moe_ag_scatter/ths_op/gemm_grouped_v3_ag_scatter.cc:249)."""
    e_cnt, n, _ = weights.shape
    out = torch.zeros(a_sorted.shape[0], n, dtype=torch.float32)
    off = routing.offsets(np.asarray(split))
    for e in range(e_cnt):
        lo, hi = int(off[e]), int(off[e + 1])
        if hi > lo:
            y = _f32(a_sorted[lo:hi]) @ _f32(weights[e]).t()
            if alpha is not None:
                y = y * float(alpha[e])
            if col_scale is not None:
                y = y * col_scale[e].to(torch.float32)[None, :]
            out[lo:hi] = y
    if row_scale is not None:
        out = out * row_scale.to(torch.float32)[:, None]
    return out * scalar


def layer0_fp32(x, weights, split, gather_idx, output_scale=None):
    """scatter_impl + gemm_impl of MoeAgScatterWithTorch (python/flux/testing/moe_ag_scatter_utils.py:207-262):
    index_select by gather_index, per-expert matmul with W[e].t(), times output_scale[e]."""
    xs = torch.index_select(x, 0, torch.as_tensor(np.asarray(gather_idx), dtype=torch.long))
    return grouped_gemm_fp32(xs, weights, split, alpha=output_scale)


def layer0_torch(x, weights, split, gather_idx, output_scale=None):
    """Same with the reference's roundings: matmul result rounded to the output dtype, then
    out.mul_(output_scale[e]) rounded again (moe_ag_scatter_utils.py:250-260)."""
    xs = torch.index_select(x, 0, torch.as_tensor(np.asarray(gather_idx), dtype=torch.long))
    out = torch.zeros(xs.shape[0], weights.shape[1], dtype=x.dtype)
    off = routing.offsets(np.asarray(split))
    for e in range(weights.shape[0]):
        lo, hi = int(off[e]), int(off[e + 1])
        if hi > lo:
            y = (_f32(xs[lo:hi]) @ _f32(weights[e]).t()).to(x.dtype)
            if output_scale is not None:
                y = (_f32(y) * float(output_scale[e])).to(x.dtype)
            out[lo:hi] = y
    return out


def topk_gather_reduce_fp32(inter, routing_idx, topk, row_weight=None, scale=1.0):
    """out[t] = scale * sum_j w[r_j] * inter[r_j], r_j = routing_idx[t*topk+j], fp32
    (src/moe_gather_rs/sm90_gemm_array_threadblock_specialized.hpp:1383-1398; weighted form
    src/moe_gather_rs/topk_gather_rs_v2.cu:394-407; loop form test/python/util/test_scatter_only.py:79-96).
    `inter` may be a list of groups, summed."""
    groups = inter if isinstance(inter, (list, tuple)) else [inter]
    idx = torch.as_tensor(np.asarray(routing_idx), dtype=torch.long).reshape(-1, topk)
    ok = (idx >= 0).to(torch.float32)
    safe = idx.clamp(min=0)
    acc = None
    for g in groups:
        rows = _f32(g)[safe]  # [T, topk, N]
        w = ok
        if row_weight is not None:
            w = w * row_weight.to(torch.float32)[safe]
        part = (rows * w[:, :, None]).sum(1)
        acc = part if acc is None else acc + part
    return acc * scale


def layer1_fp32(a_sorted, weights, split, routing_idx, topk, input_scale=None, weight_scale=None,
                output_vec_scale=None):
    """fp32 target of layer1: no intermediate rounding."""
    s = 1.0 if input_scale is None else float(input_scale.reshape(-1)[0])
    z = grouped_gemm_fp32(a_sorted, weights, split, alpha=weight_scale, row_scale=output_vec_scale, scalar=s)
    return topk_gather_reduce_fp32(z, routing_idx, topk)


def layer1_torch(a_sorted, weights, split, gather_idx, topk_idx, topk, input_scale=None, weight_scale=None,
                 output_vec_scale=None):
    """moe_gather_rs_forward_torch at world size 1 (python/flux/testing/moe_gather_rs_utils.py:26-120):
    per expert scale_v * matmul (:89; a python float times a bf16 tensor stays bf16, so the product is
    rounded), concat, times output_vec_scale and round to bf16 (:95), scatter to row
    topk*token_index + topk_index (:96-102), view(T, topk, N).sum(1) (:104).  Three roundings before the
    sum: the matmul result, the scaled result, the weighted result."""
    dt = a_sorted.dtype
    m, n = a_sorted.shape[0], weights.shape[1]
    off = routing.offsets(np.asarray(split))
    s_in = 1.0 if input_scale is None else float(input_scale.reshape(-1)[0])
    parts = []
    for e in range(weights.shape[0]):
        lo, hi = int(off[e]), int(off[e + 1])
        s_w = 1.0 if weight_scale is None else float(weight_scale[e])
        y = (_f32(a_sorted[lo:hi]) @ _f32(weights[e]).t()).to(dt)  # torch.matmul in bf16
        parts.append(((s_w * s_in) * _f32(y)).to(dt))          # scale_v * bf16 tensor -> bf16
    out = _f32(torch.cat(parts)) if parts else torch.zeros(0, n)
    if output_vec_scale is not None:
        out = out * output_vec_scale.to(torch.float32)[:, None]  # bf16 * fp32 tensor -> fp32
    out = out.to(dt)
    new_index = topk * torch.as_tensor(np.asarray(gather_idx), dtype=torch.long) + torch.as_tensor(
        np.asarray(topk_idx), dtype=torch.long)
    full = torch.zeros(m, n, dtype=dt)
    full[new_index] = out
    return full.view(m // topk, topk, n).sum(1)


def fp8_grouped_gemm_fp32(q_a, a_scale_inv, q_w, w_scale_inv, split, row_weight=None):
    """Dequantise (float(q) * scale_inv) then fp32 matmul: D[r,n] = acc * a_scale_inv[r] * w_scale_inv[e,n]
    (* row_weight[r]) — the dequant form of include/flux/args/comm_none.h:35-56 applied to e4m3 data."""
    a = q_a.to(torch.float32) * a_scale_inv.to(torch.float32)[:, None]
    w = q_w.to(torch.float32) * w_scale_inv.to(torch.float32)[:, :, None]
    return grouped_gemm_fp32(a, w, split, row_scale=row_weight)


def fp8_blockscale_grouped_gemm_fp32(q_a, a_scale, q_w, w_scale, split, block=128):
    """Block-scaled fp8 grouped GEMM, dequantise-by-block form: A[r, k] = float(q_a[r, k]) * a_scale[r, k // 128],
    W[e, n, k] = float(q_w[e, n, k]) * w_scale[e, n // 128, k // 128], then the fp32 grouped matmul.  Equal, up to
    fp32 summation order, to the promotion form of the reference's kernels and test
    (test/python/gemm_only/test_blockwise_scale_gemm_only.py:200-262: acc_per_tile = input_scale * weight_scale *
    matmul over one K block, summed over the K blocks; include/flux/args/comm_none.h:169-184).
    a_scale: [rows, K/128] (plain row-major), w_scale: [E, ceil(N/128), K/128]."""
    rows, k = q_a.shape
    e_cnt, n, _ = q_w.shape
    kb = k // block
    a = q_a.to(torch.float32).reshape(rows, kb, block) * a_scale.to(torch.float32)[:, :, None]
    w_rows = torch.repeat_interleave(w_scale.to(torch.float32), block, dim=1)[:, :n, :]      # [E, N, K/128]
    w = q_w.to(torch.float32).reshape(e_cnt, n, kb, block) * w_rows[:, :, :, None]
    return grouped_gemm_fp32(a.reshape(rows, k), w.reshape(e_cnt, n, k), split)


def a_scale_to_block128(a_scale):
    """[rows, K/128] -> the permuted layout [ceil(rows/128), K/128, 128] (row inside its block fastest) that the
    reference's quantize_vector_blockwise writes (src/quantization/ths_op/quantization.cc:75-145); rows past the end
    hold zeros."""
    rows, kb = a_scale.shape
    nb = (rows + 127) // 128
    out = torch.zeros(nb * 128, kb, dtype=a_scale.dtype)
    out[:rows] = a_scale
    return out.reshape(nb, 128, kb).permute(0, 2, 1).contiguous()


def a_scale_to_expert_k_m(a_scale, split):
    """[rows, K/128] -> experts back to back, each [K/128, rows of the expert] (rows fastest): the operand layout of
    BlockScaleGemm::forward_grouped (src/comm_none/ths_op/blockscale_gemm.cc:717-718; built the same way in
    test/python/gemm_only/test_blockwise_scale_gemm_only.py:748-753)."""
    off = routing.offsets(np.asarray(split))
    parts = [a_scale[int(off[e]):int(off[e + 1])].t().contiguous().reshape(-1) for e in range(len(split))]
    return torch.cat(parts) if parts else a_scale.reshape(-1)
