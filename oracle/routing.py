"""Routing oracle: splits, stable scatter index, gather / top-k index.  numpy int arithmetic only."""
import numpy as np


def splits(choosed, nexperts):
    """Per-expert pair count: torch.bincount(choosed.view(-1), minlength=E).int32
    (python/flux/testing/moe_utils.py:215-217).  Ids outside [0, E) are dropped pairs."""
    c = np.asarray(choosed, dtype=np.int64).reshape(-1)
    c = c[(c >= 0) & (c < nexperts)]
    return np.bincount(c, minlength=nexperts).astype(np.int32)


def offsets(split):
    """Exclusive prefix sum with the total appended (splits_cumsum of
    python/flux/testing/moe_utils.py:283-285; kernel form src/moe_ag_scatter/sort_util.cu:57-68)."""
    out = np.zeros(len(split) + 1, dtype=np.int32)
    out[1:] = np.cumsum(np.asarray(split, dtype=np.int64))
    return out


def scatter_index_stable(choosed, nexperts=None):
    """calc_scatter_index_stable (python/flux/testing/moe_utils.py:141-144):
    choosed.flatten().argsort(stable=True).argsort().int().view(shape).
    Dropped pairs (id outside [0, E)) get -1 and take no row."""
    c = np.asarray(choosed, dtype=np.int64)
    flat = c.reshape(-1)
    if nexperts is None:
        nexperts = int(flat.max()) + 1 if flat.size else 1
    valid = (flat >= 0) & (flat < nexperts)
    key = np.where(valid, flat, nexperts)  # dropped pairs sort last
    order = np.argsort(key, kind="stable")
    rank = np.empty_like(order)
    rank[order] = np.arange(flat.size)
    rank = np.where(valid, rank, -1)
    return rank.astype(np.int32).reshape(c.shape)


def scatter_index_closed_form(choosed, nexperts):
    """The same index written as its definition: offsets[e] + #{earlier flat pairs with the same e}
    (what src/cuda/moe_utils.cu:23-62 computes, with the atomic order replaced by flat order)."""
    flat = np.asarray(choosed, dtype=np.int64).reshape(-1)
    off = offsets(splits(flat, nexperts))
    seen = np.zeros(nexperts, dtype=np.int64)
    out = np.full(flat.size, -1, dtype=np.int32)
    for i, e in enumerate(flat):
        if 0 <= e < nexperts:
            out[i] = off[e] + seen[e]
            seen[e] += 1
    return out.reshape(np.asarray(choosed).shape)


def gather_index(scatter_index, topk, nrows=None):
    """Inverse permutation (python/flux/testing/moe_utils.py:96-138, kernel
    src/moe_ag_scatter/sort_util.cu:84-91): gather_index[scatter[i]] = i // topk,
    topk_index[scatter[i]] = i % topk.  Returns (gather_index, topk_index)."""
    s = np.asarray(scatter_index, dtype=np.int64).reshape(-1)
    if nrows is None:
        nrows = int((s >= 0).sum())
    g = np.zeros(nrows, dtype=np.int32)
    t = np.zeros(nrows, dtype=np.int32)
    i = np.arange(s.size)
    ok = (s >= 0) & (s < nrows)
    g[s[ok]] = (i[ok] // topk).astype(np.int32)
    t[s[ok]] = (i[ok] % topk).astype(np.int32)
    return g, t


def expert_of_row(split):
    """expert id owning each sorted row."""
    return np.repeat(np.arange(len(split), dtype=np.int32), np.asarray(split, dtype=np.int64))


def is_gather_index_stable(gather_idx, split):
    """is_gather_index_stable (python/flux/testing/moe_utils.py:278-291): strictly increasing token ids
    inside every expert segment.  Holds when no token picks the same expert twice."""
    off = offsets(split)
    g = np.asarray(gather_idx, dtype=np.int64)
    return all(bool(np.all(np.diff(g[off[e]:off[e + 1]]) > 0)) for e in range(len(split)))
