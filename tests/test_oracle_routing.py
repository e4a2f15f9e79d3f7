"""Pins oracle.routing: closed form vs library stable sort vs brute force, and the index invariants."""
import numpy as np
import pytest

from oracle import configs, routing


def brute_force_scatter(choosed, nexperts):
    flat = list(np.asarray(choosed).reshape(-1))
    pairs = sorted(range(len(flat)), key=lambda i: (flat[i], i))  # python's sort is stable, key makes it explicit
    out = [0] * len(flat)
    for pos, i in enumerate(pairs):
        out[i] = pos
    return np.array(out, dtype=np.int32).reshape(np.asarray(choosed).shape)


@pytest.mark.parametrize("tokens,topk,experts,seed", [(1, 1, 1, 0), (7, 2, 3, 1), (64, 4, 8, 2), (257, 6, 64, 3),
                                                      (100, 8, 32, 4), (33, 1, 5, 5)])
def test_scatter_index_three_ways(tokens, topk, experts, seed):
    rng = np.random.default_rng(seed)
    choosed = rng.integers(0, experts, size=(tokens, topk)).astype(np.int32)
    a = routing.scatter_index_stable(choosed, experts)
    b = routing.scatter_index_closed_form(choosed, experts)
    c = brute_force_scatter(choosed, experts)
    assert np.array_equal(a, b)
    assert np.array_equal(a, c)
    # the reference's own formula: argsort(stable).argsort()
    d = np.argsort(np.argsort(choosed.reshape(-1), kind="stable"), kind="stable").astype(np.int32)
    assert np.array_equal(a.reshape(-1), d)


def test_splits_and_offsets_closed_form():
    choosed = np.array([[0, 2], [2, 1], [2, 0], [1, 2]], dtype=np.int32)
    s = routing.splits(choosed, 4)
    assert s.tolist() == [2, 2, 4, 0]
    assert routing.offsets(s).tolist() == [0, 2, 4, 8, 8]
    si = routing.scatter_index_stable(choosed, 4)
    assert si.tolist() == [[0, 4], [5, 2], [6, 1], [3, 7]]
    g, t = routing.gather_index(si, 2)
    assert g.tolist() == [0, 2, 1, 3, 0, 1, 2, 3]
    assert t.tolist() == [0, 1, 1, 0, 1, 0, 0, 1]


@pytest.mark.parametrize("name", ["C1", "C3", "C4", "C5"])
def test_invariants_on_benchmark_routing(name):
    wl, _ = configs.make_routing(name)
    m = wl.rows
    s = wl.scatter_index.reshape(-1)
    assert wl.splits.sum() == m
    assert np.array_equal(np.sort(s), np.arange(m))  # a permutation of [0, M)
    off = routing.offsets(wl.splits)
    e = wl.choosed.numpy().reshape(-1)
    assert np.all(off[e] <= s) and np.all(s < off[e + 1])
    assert np.array_equal(wl.gather_index[s], np.arange(m) // wl.topk)
    assert np.array_equal(wl.topk_index[s], np.arange(m) % wl.topk)
    assert routing.is_gather_index_stable(wl.gather_index, wl.splits)
    assert np.array_equal(routing.expert_of_row(wl.splits)[s], e)
    # top-k weights: rows sum to one; row_weight is the same numbers in sorted-row order
    assert np.allclose(wl.topk_weight.sum(1).numpy(), 1.0, atol=1e-6)
    assert np.array_equal(wl.row_weight.numpy()[s], wl.topk_weight.numpy().reshape(-1))


def test_single_expert_is_identity():
    wl, _ = configs.make_routing("C2")
    assert np.array_equal(wl.scatter_index.reshape(-1), np.arange(wl.rows))
    assert np.array_equal(wl.gather_index, np.arange(wl.rows))
    assert wl.splits.tolist() == [4096]


def test_dropped_pairs_take_no_row():
    choosed = np.array([[0, 3], [5, 1], [-1, 0]], dtype=np.int32)  # 5 and -1 are outside [0, 4)
    si = routing.scatter_index_stable(choosed, 4)
    assert si.tolist() == [[0, 3], [-1, 2], [-1, 1]]
    assert routing.splits(choosed, 4).tolist() == [2, 1, 0, 1]
    assert np.array_equal(routing.scatter_index_closed_form(choosed, 4), si)
    g, t = routing.gather_index(si, 2)
    assert g.tolist() == [0, 2, 1, 0] and t.tolist() == [0, 1, 1, 1]


def test_empty_input():
    choosed = np.zeros((0, 2), dtype=np.int32)
    assert routing.splits(choosed, 4).tolist() == [0, 0, 0, 0]
    assert routing.scatter_index_stable(choosed, 4).shape == (0, 2)
