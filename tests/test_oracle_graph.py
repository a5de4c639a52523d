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


# ---------------------------------------------------------------- large-path segment choice (reference search_kernel.cuh:546-607)
def test_select_segments_against_numpy():
    """Ranked centroid ids while d_i / d_0 <= boundary_factor, topped up to min_segment_num, the rest 0xffffffff --
    written here from float64 distances and a stable argsort."""
    rng = np.random.default_rng(11)
    for C, dim, metric in ((7, 16, 0), (24, 32, 0), (40, 8, 0), (12, 16, 1)):
        cent = rng.standard_normal((C, dim)).astype(np.float32) * 3
        q = rng.standard_normal((200, dim)).astype(np.float32) * 3
        d = ((q[:, None].astype(np.float64) - cent[None].astype(np.float64)) ** 2).sum(-1)
        if metric == 0:
            d = np.sqrt(d)                                   # Euclidean distances are square roots everywhere (distance.cuh:22-26)
        order = np.argsort(d, 1, kind="stable")
        ds = np.take_along_axis(d, order, 1)
        for min_seg, bf in ((1, 1.0), (1, 1.3), (3, 1.15), (C, 1.05), (2, 50.0)):
            got = O.select_segments(q, cent, min_seg, bf, metric)
            ratio = ds / ds[:, :1]
            clear = (np.abs(ratio[:, 1:] - bf) > 1e-5).all(1) & (np.diff(ds, axis=1) > 1e-6 * ds[:, 1:]).all(1)   # away from ties of the two roundings
            assert clear.sum() > 150
            take = np.maximum((ratio <= bf).sum(1), min_seg)
            want = np.where(np.arange(C)[None] < take[:, None], order, INV).astype(np.uint32)
            assert np.array_equal(got[clear], want[clear]), (C, metric, min_seg, bf)
            assert (got[:, 0] == order[:, 0])[clear].all()   # the nearest partition is always listed first


# ---------------------------------------------------------------- large-path result merge (reference search_kernel.cuh:609-765)
def test_search_sub_merges_partitions_like_a_sorted_union():
    """Three partitions searched one after another into one running top-k: the result is the sorted union of each
    partition's own top-k, ids through the partition's map, whatever the order of the partitions; a partition a query does
    not list leaves its row alone, and the scan of the list stops at the first 0xffffffff.  The partitions' own top-k
    come from the small path's search (one centroid, the same start point: `get_init` with no excluded id is
    `result_init` with one centroid), so the merge is held against numpy, not against itself."""
    rng = np.random.default_rng(12)
    dim, deg, top_k, nq = 16, 8, 10, 40
    sp = O.search_params(32, deg)
    parts = []
    for s, n in enumerate((300, 180, 420)):
        data = rng.standard_normal((n, dim)).astype(np.float32) + s       # generic floats: distances are distinct
        knn, _ = O.bruteforce_knn(data, data, deg, exclude_self=True)
        mp = (rng.permutation(5000)[:n] + 10_000 * s).astype(np.uint32)
        parts.append((data, knn, mp, int(rng.integers(0, n))))
    queries = rng.standard_normal((nq, dim)).astype(np.float32) + 1
    own = []
    for data, knn, mp, start in parts:
        ids, dists, _ = O.search(data, knn, data[:1].copy(), np.array([start], np.uint32), queries, top_k, **sp)
        own.append((mp[ids], dists))
    # lists: queries 0..9 list all three, 10..19 only partitions 2 and 0, 20..29 only partition 1,
    # 30..39 list partition 1, then 0xffffffff, then partition 2 behind it (never seen: the scan stops at the gap)
    seg = np.full((nq, 3), INV, np.uint32)
    seg[:10] = [0, 1, 2]
    seg[10:20, :2] = [2, 0]
    seg[20:30, 0] = 1
    seg[30:, 0], seg[30:, 2] = 1, 2
    listed = [(0, 1, 2)] * 10 + [(0, 2)] * 10 + [(1,)] * 20
    for order in ((0, 1, 2), (2, 0, 1), (1, 2, 0)):
        fi = np.full((nq, top_k), INV, np.uint32)
        fd = np.full((nq, top_k), np.finfo(np.float32).max, np.float32)
        for s in order:
            data, knn, mp, start = parts[s]
            O.search_sub(data, knn, mp, queries, seg, s, start, top_k, sp, fi, fd)
        for q in range(nq):
            ids = np.concatenate([own[s][0][q] for s in listed[q]])
            ds = np.concatenate([own[s][1][q] for s in listed[q]])
            assert np.unique(ds).size == ds.size
            o = np.argsort(ds)[:top_k]
            assert np.array_equal(fi[q], ids[o]) and np.array_equal(fd[q], ds[o]), (order, q)


# ---------------------------------------------------------------- refine (reference graph_kernel.cuh:455-673)
def refine_model(data, graph, start, relax, p):
    """`refine_kernel` for one point, written from its definition in float64 for a beam that holds every reachable node:
    then the beam is the set reachable from the start point's neighbours (the point itself is not expanded into, but may
    sit among the start point's neighbours), sorted by distance."""
    row = graph[p]
    holes = np.nonzero(row == INV)[0]
    if holes.size == 0:
        return row.copy()
    dist = lambda a, b: np.sqrt(((data[a].astype(np.float64) - data[b].astype(np.float64)) ** 2).sum())
    seen = [int(x) for x in graph[start] if x != INV]
    todo = list(seen)
    while todo:
        u = todo.pop()
        for v in graph[u]:
            v = int(v)
            if v != INV and v != p and v not in seen:
                seen.append(v)
                todo.append(v)
    pool = sorted(seen, key=lambda x: dist(p, x))
    fills = []
    while len(fills) < holes.size and pool:
        ok = [i for i, x in enumerate(pool) if x != p and x not in row.tolist()]      # select_point: the first admissible entry
        if not ok:
            break
        h = pool[ok[0]]
        fills.append(h)
        pool = [x for x in pool[ok[0]:] if not (relax * dist(h, x) < dist(p, x))]       # entries before the head are dropped too
    out = row.copy()
    out[holes[:len(fills)]] = fills
    return out


BIG_BEAM = dict(beam=64, max_iterations=4000, min_iterations=0, hash_bit=12, hash_reset_interval=1 << 20)


def test_refine_hand_built_line_graph():
    """Twelve points on a line with growing gaps.  With relaxant 1 a chosen neighbour removes everything behind it on its
    side of the point and nothing on the other side, so a row gets the nearest admissible point, then the nearest
    admissible farther point on the other side, and nothing more."""
    x = np.cumsum([0, 1, 1.1, 1.2, 1.3, 1.4, 1.5, 1.6, 1.7, 1.8, 1.9, 2.0])
    data = np.zeros((12, 4), np.float32)
    data[:, 0] = x
    g = np.full((12, 4), INV, np.uint32)
    for i in range(12):
        g[i, 0] = i + 1 if i < 11 else 10
        g[i, 1] = i - 1 if i > 0 else 5          # row 0 (the start point) also names 5: point 5 meets itself in its beam
    full = g.copy()
    full[:, 2], full[:, 3] = (np.arange(12) + 2) % 12, (np.arange(12) + 3) % 12   # rows without holes
    g[3] = full[3]
    g[5] = [6, INV, 4, INV]                      # holes at slots 1 and 3
    g[8] = [9, 7, 10, INV]                       # one hole
    g[2, 1] = INV                                # row 2 = [3, INV, INV, INV]: three holes, only two points can be chosen
    cent, sps = data[:1].copy(), np.array([0], np.uint32)
    got, _ = O.refine(data, g, cent, sps, BIG_BEAM, 1.0)
    assert np.array_equal(got[3], g[3])                                   # no hole: untouched
    # point 5 (x = 6.0): by distance 4 (1.4, in the row), 6 (1.5, in the row), 3 (2.7) <- first admissible; behind it on
    # the left 2, 1, 0 fall, on the right 7 (3.1) is the next head; after it nothing is left.  5 itself (distance 0, from
    # the start point's row) is skipped.
    assert got[5].tolist() == [6, 3, 4, 7]
    # point 8 (x = 10.8): 7 and 9 are in the row, 10 is in the row, 6 (3.3) is the first admissible; one hole, one pick
    assert got[8].tolist() == [9, 7, 10, 6]
    # point 2 (x = 2.1): 1 (1.1) first, then 3 (1.2) is in the row -> 4 (2.5); the third hole stays empty
    assert got[2].tolist() == [3, 1, 4, INV]
    for p in range(12):
        assert np.array_equal(got[p], refine_model(data, g, 0, 1.0, p)), p


def test_refine_against_definition_on_random_graphs():
    rng = np.random.default_rng(13)
    for n, deg, relax in ((60, 4, 1.05), (150, 8, 1.05), (150, 8, 1.3)):
        data = rng.standard_normal((n, 8)).astype(np.float32)
        g, _ = O.bruteforce_knn(data, data, deg, exclude_self=True)
        g = np.ascontiguousarray(g[:, rng.permutation(deg)])
        g[rng.random((n, deg)) < 0.35] = INV
        g[0, 0] = 7                                                       # the start point's row is not empty
        sp = dict(BIG_BEAM, beam=256)
        got, _ = O.refine(data, g, data[:1].copy(), np.array([0], np.uint32), sp, relax)
        dist = lambda a, b: np.sqrt(((data[a].astype(np.float64) - data[b].astype(np.float64)) ** 2).sum())
        for p in range(n):
            assert np.array_equal(got[p], refine_model(data, g, 0, relax, p)), (n, p)
            old, new = g[p], got[p]
            assert ((new == old) | (old == INV)).all()                    # only holes change
            added = new[(old == INV) & (new != INV)].tolist()
            assert p not in added and not set(added) & set(old.tolist()) and len(set(added)) == len(added)
            for i, a in enumerate(added):                                 # no chosen neighbour occludes a later one
                for b in added[i + 1:]:
                    assert relax * dist(a, b) >= dist(p, b) * (1 - 1e-6)
            holes = np.nonzero(old == INV)[0]
            assert (new[holes[len(added):]] == INV).all()                 # filled in slot order, front first


# ---------------------------------------------------------------- visited-set reset and restore (reference search_kernel.cuh:327-334,438-469)
def path_with_far_node(n):
    """Nodes 0..n-1 at x = 0..n-1, node i -> (i + 1, F); F = node n far away on the other side.  Query beyond the last node."""
    data = np.zeros((n + 1, 4), np.float32)
    data[:n, 0] = np.arange(n)
    data[n, 0] = -1000.0
    g = np.full((n + 1, 2), INV, np.uint32)
    g[:n, 0] = np.arange(1, n + 1)
    g[n - 1, 0] = INV
    g[:n, 1] = n
    q = np.zeros((1, 4), np.float32)
    q[0, 0] = n - 1 + 0.25
    return data, g, q


def test_hash_reset_and_restore_on_a_path():
    """Hand-derived run.  The search enters at node 1 and F (the neighbours of start point 0) and walks one node per
    iteration: iteration j expands node j + 1.  The beam (32) holds F until 32 path nodes are known, i.e. until the merge
    at the top of iteration 31.  A reset empties the visited set and the restore puts the beam back, so from then on F is
    forgotten by every reset and scored once more by the expansion that follows it; path nodes in the beam never are.
    Rows scored = n path nodes... minus the start point (never scored) + F once + one per reset in iterations 31..n-2.
    The table has 64 slots: without the clearing it overflows after 64 nodes and the walk stops; without the restore the
    node behind the parent would be scored again on every step."""
    n = 120
    data, g, q = path_with_far_node(n)
    cent, sps = data[:1].copy(), np.array([0], np.uint32)
    want_ids = np.arange(n - 1, n - 11, -1)
    want_d = (q[0, 0] - np.arange(n - 1, n - 11, -1)).astype(np.float32)
    for reset in (1, 2, 3, 5, 7, 1 << 20):
        hash_bit = 6 if reset <= 7 else 10
        ids, dists, st = O.search(data, g, cent, sps, q, 10, 32, 1000, 0, hash_bit, reset)
        assert ids[0].tolist() == want_ids.tolist() and np.array_equal(dists[0], want_d), reset
        resets_after_eviction = sum(1 for j in range(31, n - 1) if (j + 1) % reset == 0)
        assert st["iterations"] == n, (reset, st)
        assert st["graph_rows"] == n, (reset, st)                       # the start point's row + one row per expanded node 1..n-1
        assert st["rows_scored"] == (n - 1) + 1 + resets_after_eviction, (reset, st)


def test_hash_reset_every_iteration_returns_no_id_twice():
    rng = np.random.default_rng(14)
    data = rng.standard_normal((3000, 16)).astype(np.float32)
    knn, _ = O.bruteforce_knn(data, data, 16, exclude_self=True)
    queries = rng.standard_normal((100, 16)).astype(np.float32)
    cent, sps = data[:1].copy(), np.array([17], np.uint32)
    base = O.search(data, knn, cent, sps, queries, 32, 64, 400, 0, 13, 1 << 20)
    for reset in (1, 2, 3):
        ids, dists, st = O.search(data, knn, cent, sps, queries, 32, 64, 400, 0, 8, reset)
        for row in ids:
            assert np.unique(row).size == row.size
        # a forgotten node is farther than everything the beam held when it left, so scoring it again changes nothing
        assert np.array_equal(ids, base[0]) and np.array_equal(dists, base[1])
        assert st["rows_scored"] > base[2]["rows_scored"] and st["iterations"] == base[2]["iterations"]


def test_nnd_oracle_from_given_start_lists():
    """The build from caller-supplied start lists (what pairs the GPU and CPU sides of the pipeline comparison) is the
    same algorithm: same recall as the build from shuffled lists, valid structure, and it does depend on the lists."""
    from glide_amd.datasets import recall
    rng = np.random.default_rng(15)
    data = lowdim_data(4000, 128, seed=9)
    seg_start, seg_len = np.array([0, 2500], np.uint32), np.array([2500, 1500], np.uint32)
    for k in (32, 64):
        width = O.nnd_extended_degree(k)
        num_sub = width // 32

        def lists(seed):
            r = np.random.default_rng(seed)
            out = np.empty((4000, width), np.int32)
            for s, l in ((0, 2500), (2500, 1500)):
                for sub in range(num_sub):       # sub-list `sub` holds ids congruent to sub modulo num_sub
                    pool = np.arange(sub, l, num_sub)
                    out[s:s + l, sub * 32:(sub + 1) * 32] = r.choice(pool, (l, 32))
            return out

        a = O.nnd_build_from(data, seg_start, seg_len, k, 8, lists(1)).astype(np.uint32)
        b = O.nnd_build_from(data, seg_start, seg_len, k, 8, lists(1)).astype(np.uint32)
        c = O.nnd_build_from(data, seg_start, seg_len, k, 8, lists(2)).astype(np.uint32)
        ref = O.nnd_build(data, seg_start, seg_len, k, 8).astype(np.uint32)
        for s, l in ((0, 2500), (2500, 1500)):
            assert (a[s:s + l] < l).all()
            gt, _ = O.bruteforce_knn(data[s:s + l], data[s:s + 200], 32, exclude_self=True)
            ra, rr = recall(a[s:s + 200, :32], gt, 32), recall(ref[s:s + 200, :32], gt, 32)
            assert abs(ra - rr) <= 0.01 and ra >= 0.9, (k, ra, rr)
        assert not np.array_equal(a, c)
        assert (np.sort(a, 1) == np.sort(b, 1)).mean() > 0.99      # the same lists in, the same graph out up to thread timing
