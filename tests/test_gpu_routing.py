"""GPU parity, routing: indices and splits must be bit-exact against the CPU oracle (stable order)."""
import hashlib
import json
import os

import numpy as np
import pytest
import torch

from oracle import configs, routing

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_route_sort(choosed_np, experts):
    from flux_amd import capi
    c = torch.from_numpy(np.ascontiguousarray(choosed_np)).cuda()
    splits, offsets, scatter, gather, tki = capi.route_sort(c, experts)
    torch.cuda.synchronize()
    return [t.cpu().numpy() for t in (splits, offsets, scatter, gather, tki)]


def check(choosed_np, experts, topk):
    splits, offsets, scatter, gather, tki = run_route_sort(choosed_np, experts)
    ref_splits = routing.splits(choosed_np, experts)
    ref_scatter = routing.scatter_index_stable(choosed_np, experts)
    nrows = int(ref_splits.sum())
    ref_gather, ref_tki = routing.gather_index(ref_scatter, topk, nrows)
    assert np.array_equal(splits, ref_splits)
    assert np.array_equal(offsets, routing.offsets(ref_splits))
    assert np.array_equal(scatter, ref_scatter)
    assert np.array_equal(gather[:nrows], ref_gather)
    assert np.array_equal(tki[:nrows], ref_tki)


@pytest.mark.parametrize("name", ["C1", "C2", "C3", "C4", "C5"])
def test_benchmark_routing_bit_exact(name):
    wl, _ = configs.make_routing(name)
    print(f"[case] route_sort {name} T={wl.tokens} k={wl.topk} E={wl.experts}", flush=True)
    check(wl.choosed.numpy(), wl.experts, wl.topk)


def test_golden_fixture_and_hashes():
    z = np.load(os.path.join(ROOT, "tests", "golden", "routing_c1.npz"))
    splits, offsets, scatter, gather, tki = run_route_sort(z["choosed"], 8)
    assert np.array_equal(splits, z["splits"]) and np.array_equal(scatter, z["scatter_index"])
    assert np.array_equal(gather, z["gather_index"]) and np.array_equal(tki, z["topk_index"])
    want = json.load(open(os.path.join(ROOT, "tests", "golden", "index_hashes.json")))
    sha = lambda a: hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()
    for name, h in want.items():
        wl, _ = configs.make_routing(name)
        splits, offsets, scatter, gather, tki = run_route_sort(wl.choosed.numpy(), wl.experts)
        assert splits.tolist() == h["splits"]
        assert sha(scatter) == h["scatter_index"] and sha(gather) == h["gather_index"] and sha(tki) == h["topk_index"]


@pytest.mark.parametrize("tokens,topk,experts,seed", [
    (1, 1, 1, 0), (3, 2, 5, 1), (63, 1, 2, 2), (64, 8, 9, 3), (513, 1, 3, 4), (2048, 2, 8, 5),
    (2049, 3, 65, 6), (5000, 7, 130, 7), (40000, 2, 1024, 8), (300, 4, 1000, 9)])
def test_random_and_ragged_shapes(tokens, topk, experts, seed):
    rng = np.random.default_rng(seed)
    print(f"[case] route_sort random T={tokens} k={topk} E={experts}", flush=True)
    choosed = rng.integers(0, experts, size=(tokens, topk)).astype(np.int32)
    check(choosed, experts, topk)


def test_all_pairs_one_expert_and_empty_experts():
    choosed = np.full((3000, 2), 5, dtype=np.int32)
    check(choosed, 8, 2)
    choosed = (np.arange(4000).reshape(2000, 2) % 2 * 7).astype(np.int32)  # only experts 0 and 7 used
    check(choosed, 8, 2)


def test_dropped_pairs():
    rng = np.random.default_rng(11)
    choosed = rng.integers(-1, 10, size=(1500, 4)).astype(np.int32)  # -1, 8 and 9 are outside [0, 8)
    check(choosed, 8, 4)


def test_empty_input():
    check(np.zeros((0, 2), dtype=np.int32), 4, 2)


def test_gather_index_entry_point():
    from flux_amd import capi
    wl, _ = configs.make_routing("C4")
    s = torch.from_numpy(wl.scatter_index).cuda()
    g, t = capi.gather_index(s, wl.topk)
    assert np.array_equal(g.cpu().numpy(), wl.gather_index)
    assert np.array_equal(t.cpu().numpy(), wl.topk_index)


def test_full_size_properties():
    """Size-independent properties on a shape larger than any benchmark config (1M pairs, 256 experts)."""
    rng = np.random.default_rng(12)
    tokens, topk, experts = 131072, 8, 256
    choosed = rng.integers(0, experts, size=(tokens, topk)).astype(np.int32)
    splits, offsets, scatter, gather, tki = run_route_sort(choosed, experts)
    m = tokens * topk
    s = scatter.reshape(-1)
    assert splits.sum() == m and offsets[-1] == m
    assert np.array_equal(np.sort(s), np.arange(m))
    assert np.array_equal(gather[s], np.arange(m) // topk) and np.array_equal(tki[s], np.arange(m) % topk)
    e = choosed.reshape(-1)
    assert np.all(offsets[e] <= s) and np.all(s < offsets[e + 1])
    order = np.argsort(s)
    assert np.all(np.diff(e[order]) >= 0)  # sorted by expert
    same = np.diff(e[order]) == 0
    assert np.all(np.diff(order)[same] > 0)  # stable inside an expert
