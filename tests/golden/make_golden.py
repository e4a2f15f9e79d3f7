"""Writes the committed golden fixtures from the CPU oracle (run from the repo root:
`python tests/golden/make_golden.py`).  The reference holds no golden vectors for this path, so these
pin the oracle's own outputs against later drift; the oracle itself is pinned in tests/test_oracle_*.py.

  routing_c1.npz       C1 routing arrays (choosed, splits, scatter/gather/topk index)
  quant_16x256.npz     a 16x256 bf16 matrix with its per-row and 1x128-block e4m3 codes and scales
  index_hashes.json    sha256 of the C3 / C4 / C5 routing arrays (tensors too large to commit)
"""
import hashlib
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import configs, quant  # noqa: E402


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def main():
    wl, _ = configs.make_routing("C1")
    np.savez_compressed(os.path.join(HERE, "routing_c1.npz"), choosed=wl.choosed.numpy(), splits=wl.splits,
                        scatter_index=wl.scatter_index, gather_index=wl.gather_index, topk_index=wl.topk_index,
                        topk_weight=wl.topk_weight.numpy())

    g = torch.Generator().manual_seed(4242)
    x = torch.randn(16, 256, generator=g) * torch.logspace(-3, 2, 16)[:, None]
    x[3] = 0
    x[5, 7] = 1e30
    bits = x.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    q_row, s_row = quant.quant_rows_c(bits, 0, 0.0, False)
    q_blk, s_blk = quant.quant_rows_c(bits, 128, 0.0, True)
    np.savez_compressed(os.path.join(HERE, "quant_16x256.npz"), x_bits=bits, q_row=q_row, scale_inv_row=s_row,
                        q_blk=q_blk, scale_inv_blk_perm=s_blk)

    hashes = {}
    for name in ("C3", "C4", "C5"):
        wl, _ = configs.make_routing(name)
        hashes[name] = {"choosed": sha(wl.choosed.numpy()), "splits": wl.splits.tolist(),
                        "scatter_index": sha(wl.scatter_index), "gather_index": sha(wl.gather_index),
                        "topk_index": sha(wl.topk_index)}
    with open(os.path.join(HERE, "index_hashes.json"), "w") as f:
        json.dump(hashes, f, indent=1)


if __name__ == "__main__":
    main()
