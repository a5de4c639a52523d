"""Pins of the CPU oracle's graph-stage functions: hand-worked cases, invariants and brute force in float64."""
import numpy as np
import pytest

from conftest import lowdim_data
from oracle import oracle as O

INV = 0xFFFFFFFF


# ---------------------------------------------------------------- prune (reference graph_kernel.cuh:70-143)
def prune_float64(data, pool_ids, pool_dists, degree, relax):
    """Greedy relaxed-RNG selection written from the definition, in float64."""
    pool = list(zip(pool_ids.tolist(), pool_dists.tolist()))
    out = []
    while len(out) < degree and pool:
        h = pool[0][0]
        out.append(h)
        nxt = []
        for i, di in pool[1:]:
            dhi = np.sqrt(((data[h].astype(np.float64) - data[i].astype(np.float64)) ** 2).sum())
            if not (relax * dhi < di):
                nxt.append((i, di))
        pool = nxt
    return out


def test_prune_matches_definition_and_invariant():
    rng = np.random.default_rng(0)
    data = lowdim_data(400, 128, seed=3)
    for trial in range(30):
        p = int(rng.integers(0, 400))
        ids = rng.permutation(400)[:48]
        ids = ids[ids != p]
        d = np.sqrt(((data[ids].astype(np.float64) - data[p].astype(np.float64)) ** 2).sum(1)).astype(np.float32)
        order = np.argsort(d, kind="stable")
        ids, d = ids[order].astype(np.uint32), d[order]
        got, n = O.prune(data, 0, ids, d, 16, 1.05)
        want = prune_float64(data, ids, d, 16, 1.05)
        assert got[:n].tolist() == want, trial
        assert (got[n:] == INV).all()
        # invariant: no kept neighbour occludes a later kept one
        dist = lambda a, b: np.sqrt(((data[a].astype(np.float64) - data[b].astype(np.float64)) ** 2).sum())
        dp = dict(zip(ids.tolist(), d.tolist()))
        for a_i, a in enumerate(want):
            for b in want[a_i + 1:]:
                assert 1.05 * dist(a, b) >= dp[b] * (1 - 1e-6)


def test_prune_segment_offset_and_small_pools():
    data = lowdim_data(100, 128, seed=4)
    ids = np.array([3, 7, 9], np.uint32)                      # local ids; rows live at +50
    d = np.sqrt(((data[ids + 50].astype(np.float64) - data[0].astype(np.float64)) ** 2).sum(1)).astype(np.float32)
    order = np.argsort(d)
    got, n = O.prune(data, 50, ids[order], d[order], 8, 1.05)
    assert n >= 1 and got[0] == ids[order][0] + 50 and set(got[:n].tolist()) <= set((ids + 50).tolist())
    got, n = O.prune(data, 0, np.array([], np.uint32), np.array([], np.float32), 8, 1.05)
    assert n == 0 and (got == INV).all()


# ---------------------------------------------------------------- boundary merge (reference graph_kernel.cuh:160-247)
def test_merge_boundary_row_hand_worked():
    mp = np.arange(100, dtype=np.uint32) + 1000               # reorder id r -> original id 1000 + r
    # D = 8.  Row has 5 entries + 3 empty; copy proposes 4 neighbours of which 1 repeats (1002) -> dups 1 < D/2 = 4:
    # need = min(3 fresh, 4 - 1) = 3; walk from the tail: slots 7,6,5 are empty -> fresh[0..2] land there in that order.
    row = np.array([1001, 1002, 1003, 1004, 1005, INV, INV, INV], np.uint32)
    nb = np.array([2, 10, 11, 12, INV, INV, INV, INV], np.uint32)
    assert O.merge_boundary_row(row, nb, mp).tolist() == [1001, 1002, 1003, 1004, 1005, 1012, 1011, 1010]
    # full row, no repeats: need = min(3, 4) = 3 -> overwrite the tail slots 7,6,5
    row = np.array([1001, 1002, 1003, 1004, 1005, 1006, 1007, 1008], np.uint32)
    nb = np.array([20, 21, 22, INV, INV, INV, INV, INV], np.uint32)
    assert O.merge_boundary_row(row, nb, mp).tolist() == [1001, 1002, 1003, 1004, 1005, 1022, 1021, 1020]
    # repeated entries are protected: dups at slots 6 and 7 -> tail walk skips them and overwrites 5 and 4
    row = np.array([1001, 1002, 1003, 1004, 1005, 1006, 1007, 1008], np.uint32)
    nb = np.array([7, 8, 30, 31, 32, INV, INV, INV], np.uint32)            # 1007, 1008 repeat; need = min(3, 4 - 2) = 2
    assert O.merge_boundary_row(row, nb, mp).tolist() == [1001, 1002, 1003, 1004, 1031, 1030, 1007, 1008]
    # many repeats (>= D/2): only empty slots are filled, front to back
    row = np.array([1001, 1002, 1003, 1004, 1005, INV, INV, INV], np.uint32)
    nb = np.array([1, 2, 3, 4, 40, 41, 42, 43], np.uint32)                 # 4 repeats, 4 fresh, 3 holes
    assert O.merge_boundary_row(row, nb, mp).tolist() == [1001, 1002, 1003, 1004, 1005, 1040, 1041, 1042]
    # nothing proposed: unchanged
    row = np.array([1001, INV, INV, INV, INV, INV, INV, INV], np.uint32)
    assert O.merge_boundary_row(row, np.full(8, INV, np.uint32), mp).tolist() == row.tolist()


# ---------------------------------------------------------------- reverse edges (reference graph_kernel.cuh:378-453)
def reverse_python(g):
    n, D = g.shape
    rev = [[] for _ in range(n)]
    for c in range(D):
        for s in range(n):
            t = int(g[s, c])
            if t < n and s not in g[t].tolist():
                rev[t].append(s)
    out = g.copy()
    for p in range(n):
        take = rev[p][:D]
        k = 0
        for i in range(D):
            if out[p, i] == INV and k < len(take):
                out[p, i] = take[k]
                k += 1
    return out


def test_reverse_edges_brute_force():
    rng = np.random.default_rng(1)
    for n, D in ((60, 4), (200, 8), (300, 32)):
        g = rng.integers(0, n, (n, D)).astype(np.uint32)
        g[rng.random((n, D)) < 0.5] = INV
        g[:, 0] = 5 % n                                   # a hub: more reverse edges than slots
        got = O.reverse_edges(g)
        assert np.array_equal(got, reverse_python(g))
        assert ((got == g) | (g == INV)).all()            # only empty slots change


# ---------------------------------------------------------------- partition (reference partition_kernel.cuh:22-100)
def test_partition_assign_float64_and_reorder():
    data = lowdim_data(3000, 128, seed=6)
    rng = np.random.default_rng(2)
    cent = data[rng.permutation(3000)[:12]] + rng.standard_normal((12, 128)).astype(np.float32) * 2
    idx, lens, near = O.partition_assign(data, cent, 1.08)
    d = np.sqrt(((data[:, None].astype(np.float64) - cent[None].astype(np.float64)) ** 2).sum(-1))
    order = np.argsort(d, 1)
    d0, d1 = d[np.arange(3000), order[:, 0]], d[np.arange(3000), order[:, 1]]
    clear = d1 / d0 - 1 > 1e-5
    assert np.array_equal(idx[clear, 0], order[clear, 0])
    far = np.abs(d1 / d0 - 1.08) > 1e-5
    assert np.array_equal((idx[:, 2] != INV)[far & clear], (d1 / d0 <= 1.08)[far & clear])
    assert np.allclose(near[:, 0], d0, rtol=1e-5) and lens[:12].sum() == 3000
    for s in range(12):
        m = np.nonzero(idx[:, 0] == s)[0]
        assert np.array_equal(idx[m, 1], np.arange(m.size))
    starts = O.segment_starts(lens)
    rn = 3000 + int(lens[12])
    rdata, mp = O.reorder(data, idx, starts, rn)
    assert np.array_equal(rdata, data[mp]) and sorted(mp[:3000].tolist()) == list(range(3000))
    assert np.array_equal(np.sort(mp[3000:]), np.nonzero(idx[:, 2] != INV)[0])
    # one centroid: no boundary list at all
    idx1, lens1, _ = O.partition_assign(data[:100], cent[:1], 1.5)
    assert lens1.tolist() == [100, 0] and (idx1[:, 2] == INV).all()


# ---------------------------------------------------------------- whole chain
def test_pipeline_search_recall_and_structure(small_index):
    from glide_amd.datasets import recall
    idx = small_index
    g = idx["graph"]
    n = g.shape[0]
    valid = g != INV
    assert (g[valid] < n).all()
    for row in g[:200]:                                      # no repeated neighbour in a row
        r = row[row != INV]
        assert len(set(r.tolist())) == r.size
    gt, _ = O.bruteforce_knn(idx["data"], idx["queries"], 10)
    sp = O.search_params(64, 32)
    ids, dists, st = O.search(idx["data"], g, idx["centroids"], idx["start_points"], idx["queries"], 10, **sp)
    assert recall(ids, gt, 10) >= 0.97
    assert (np.diff(dists, axis=1) >= 0).all()               # results come out ascending
    exact = np.sqrt(((idx["data"][ids[:50].astype(np.int64)].astype(np.float64) - idx["queries"][:50, None].astype(np.float64)) ** 2).sum(-1))
    assert np.allclose(dists[:50], exact, rtol=1e-6)
    assert st["iterations"] <= 71 * 300 and st["graph_rows"] <= st["iterations"]


def test_nnd_oracle_recall():
    from glide_amd.datasets import recall
    data = lowdim_data(5000, 128, seed=8)
    seg_start, seg_len = np.array([0, 3000], np.uint32), np.array([3000, 2000], np.uint32)
    knn = O.nnd_build(data, seg_start, seg_len, 32, 8).astype(np.uint32)
    for s, l in ((0, 3000), (3000, 2000)):
        assert (knn[s:s + l] < l).all()
        gt, _ = O.bruteforce_knn(data[s:s + l], data[s:s + 200], 32, exclude_self=True)
        assert recall(knn[s:s + 200], gt, 32) >= 0.97


def test_bruteforce_matches_numpy():
    rng = np.random.default_rng(3)
    data, q = rng.standard_normal((500, 16)).astype(np.float32), rng.standard_normal((20, 16)).astype(np.float32)
    ids, d = O.bruteforce_knn(data, q, 5)
    full = ((data[None].astype(np.float64) - q[:, None].astype(np.float64)) ** 2).sum(-1)
    assert np.array_equal(ids, np.argsort(full, 1)[:, :5])
    assert np.allclose(d, np.sqrt(np.sort(full, 1)[:, :5]), rtol=1e-5)
