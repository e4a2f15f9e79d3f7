"""Seeded synthetic workloads C1..C5 (the benchmark configurations) — test / bench infrastructure.

Everything is generated on the CPU from torch.Generator().manual_seed(1000 + index), so the GPU path and
the CPU oracle see identical bits.  Weights are stored [E, N, K] (K contiguous), the layout the
reference's ops take (src/moe_ag_scatter/ths_op/gemm_grouped_v3_ag_scatter.cc:249,
src/moe_gather_rs/ths_op/gemm_grouped_v3_gather_rs.cc:638); the math is x @ W[e].T.
"""
from dataclasses import dataclass, field

import numpy as np
import torch

from . import routing

SHAPES = {
    # name: (index, tokens, topk, experts, hidden, ffn, dtype, routing)
    "C1": (1, 256, 2, 8, 1024, 2048, "bf16", "softmax"),
    "C2": (2, 4096, 1, 1, 6144, 12288, "bf16", "single"),
    "C3": (3, 8192, 2, 8, 4096, 14336, "bf16", "softmax"),
    "C4": (4, 16384, 6, 64, 2048, 1408, "bf16", "zipf"),
    "C5": (5, 4096, 8, 32, 7168, 2048, "fp8", "uniform"),
}


@dataclass
class Workload:
    name: str
    tokens: int
    topk: int
    experts: int
    hidden: int
    ffn: int
    dtype: str
    choosed: torch.Tensor            # [T, k] int32
    topk_weight: torch.Tensor        # [T, k] fp32, rows sum to 1
    splits: np.ndarray = None        # [E] int32
    scatter_index: np.ndarray = None  # [T, k] int32
    gather_index: np.ndarray = None  # [M] int32
    topk_index: np.ndarray = None    # [M] int32
    row_weight: torch.Tensor = None  # [M] fp32, top-k weight of each sorted row (Flux: output_vec_scale)
    tensors: dict = field(default_factory=dict)

    @property
    def rows(self):
        return self.tokens * self.topk


def _routing(kind, tokens, topk, experts, gen):
    if kind == "single":
        choosed = torch.zeros(tokens, topk, dtype=torch.int32)
        weight = torch.ones(tokens, topk, dtype=torch.float32)
        return choosed, weight
    logits = torch.randn(tokens, experts, generator=gen, dtype=torch.float32)
    if kind == "softmax":
        # softmax over N(0,1) logits, top-k, weights renormalised to sum 1.
        probs = torch.softmax(logits, dim=-1)
        weight, idx = torch.topk(probs, topk, dim=-1)
    else:
        if kind == "zipf":
            p = (torch.arange(1, experts + 1, dtype=torch.float64) ** -1.2).to(torch.float32)
        else:  # uniform assignment without replacement
            p = torch.ones(experts, dtype=torch.float32)
        idx = torch.multinomial(p.repeat(tokens, 1), topk, replacement=False, generator=gen)
        weight = torch.softmax(torch.gather(logits, 1, idx), dim=-1)
    weight = weight / weight.sum(dim=-1, keepdim=True)
    return idx.to(torch.int32), weight.to(torch.float32)


def make_routing(name, tokens=None):
    idx, t, k, e, h, f, dtype, kind = SHAPES[name]
    if tokens is not None:
        t = tokens
    gen = torch.Generator().manual_seed(1000 + idx)
    choosed, weight = _routing(kind, t, k, e, gen)
    wl = Workload(name, t, k, e, h, f, dtype, choosed, weight)
    c = choosed.numpy()
    wl.splits = routing.splits(c, e)
    wl.scatter_index = routing.scatter_index_stable(c, e)
    wl.gather_index, wl.topk_index = routing.gather_index(wl.scatter_index, k, t * k)
    rw = torch.empty(t * k, dtype=torch.float32)
    rw[torch.as_tensor(wl.scatter_index.reshape(-1), dtype=torch.long)] = weight.reshape(-1)
    wl.row_weight = rw
    return wl, gen


def _randn_bf16(shape, std, gen):
    out = torch.empty(shape, dtype=torch.bfloat16)
    flat = out.view(-1)
    step = 1 << 26
    for lo in range(0, flat.numel(), step):  # chunked: no full-size fp32 temporary
        n = min(step, flat.numel() - lo)
        flat[lo:lo + n] = (torch.randn(n, generator=gen, dtype=torch.float32) * std).to(torch.bfloat16)
    return out


def make_workload(name, tokens=None, hidden=None, ffn=None, with_w2=True):
    """Routing + activations N(0,1) + weights N(0,0.02), all bf16.  `tokens/hidden/ffn` shrink the shape
    (same distributions) for cases the CPU oracle must finish in seconds."""
    wl, gen = make_routing(name, tokens)
    if hidden is not None:
        wl.hidden = hidden
    if ffn is not None:
        wl.ffn = ffn
    t, k, e, h, f = wl.tokens, wl.topk, wl.experts, wl.hidden, wl.ffn
    wl.tensors["x"] = _randn_bf16((t, h), 1.0, gen)
    wl.tensors["w1"] = _randn_bf16((e, f, h), 0.02, gen)         # layer0: [E, N=F, K=H]
    if with_w2:
        wl.tensors["w2"] = _randn_bf16((e, h, f), 0.02, gen)     # layer1: [E, N=H, K=F]
        wl.tensors["act"] = _randn_bf16((t * k, f), 1.0, gen)    # independent layer1 input
    return wl
