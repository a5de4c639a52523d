"""Large-path kernels (one staged partition at a time) against the CPU oracle."""
import numpy as np
import pytest

from conftest import lowdim_data

pytestmark = pytest.mark.gpu
INV = 0xFFFFFFFF


@pytest.fixture(scope="module")
def hip():
    from glide_amd import capi
    capi.set_device(0)
    return capi


@pytest.fixture(scope="module")
def large_index():
    """Three partitions without a boundary list, built by the oracle's large-path functions."""
    from oracle import oracle as O
    data = lowdim_data(7000, 128, seed=41)
    queries = lowdim_data(250, 128, seed=42)
    cent = O.kmeans(data[::3], 3, iterations=8)
    idx, lens, _ = O.partition_assign(data, cent, 0.0)             # factor 0: nobody is a boundary point
    assert lens[3] == 0
    starts = O.segment_starts(lens)
    rdata, mp = O.reorder(data, idx, starts, 7000)
    knn = O.nnd_build(rdata, starts[:3], lens[:3], 32, 6).astype(np.uint32)
    sp_b, sp_r = O.search_params(64, 32), O.search_params(128, 32)
    rng = np.random.default_rng(0)
    start_points = np.array([rng.integers(0, l) for l in lens[:3]], np.uint32)
    segs = []
    for s in range(3):
        a, l = int(starts[s]), int(lens[s])
        g0, st0 = O.build_segment(rdata[a:a + l], knn[a:a + l], int(start_points[s]), 32, sp_b, 1.05)
        g1 = O.reverse_edges(g0)
        g2, st2 = O.refine_segment(rdata[a:a + l], g1, int(start_points[s]), sp_r, 1.05)
        segs.append(dict(data=rdata[a:a + l], knn=knn[a:a + l], map=mp[a:a + l], built=g0, st_built=st0, rev=g1, graph=g2, st_ref=st2))
    return dict(data=data, queries=queries, cent=cent, segs=segs, start_points=start_points, sp_b=sp_b, sp_r=sp_r)


def test_build_and_refine_segment_bit_exact(hip, large_index):
    L = large_index
    for s, seg in enumerate(L["segs"]):
        n = seg["data"].shape[0]
        d_data, d_knn = hip.DeviceArray.from_numpy(seg["data"]), hip.DeviceArray.from_numpy(seg["knn"])
        g = hip.DeviceArray.full((n, 32), 0xDEADBEEF)
        cnt = hip.new_counters()
        p = L["sp_b"]
        hip.build_segment(d_data, n, 128, d_knn, 32, int(L["start_points"][s]), 32, p["beam"], p["max_iterations"], p["min_iterations"],
                          p["hash_bit"], p["hash_reset_interval"], 1.05, 0, g, cnt)
        hip.synchronize()
        assert np.array_equal(g.numpy(), seg["built"])
        st = seg["st_built"]
        assert hip.read_counters(cnt) == [st["iterations"], st["rows_scored"], st["graph_rows"]]
        g_in, g_out = hip.DeviceArray.from_numpy(seg["rev"]), hip.DeviceArray.full((n, 32), 0xDEADBEEF)
        p = L["sp_r"]
        hip.refine_segment(d_data, n, 128, g_in, g_out, 32, int(L["start_points"][s]), p["beam"], p["max_iterations"], p["min_iterations"],
                           p["hash_bit"], p["hash_reset_interval"], 1.05, 0)
        hip.synchronize()
        assert np.array_equal(g_out.numpy(), seg["graph"])


@pytest.mark.parametrize("c,min_seg,bf", [(3, 1, 1.2), (3, 2, 1.0), (40, 3, 1.1), (200, 5, 1.05), (7, 7, 1.0)])
def test_select_segments_bit_exact(hip, c, min_seg, bf):
    from oracle import oracle as O
    data = lowdim_data(3000, 128, seed=c)
    queries = np.rint(lowdim_data(200, 128, seed=c + 1))
    cent = np.rint(data[np.random.default_rng(c).permutation(3000)[:c]])        # integer centroids: exact distances
    want = O.select_segments(queries, cent, min_seg, bf)
    d_q, d_c = hip.DeviceArray.from_numpy(queries), hip.DeviceArray.from_numpy(cent)
    out = hip.DeviceArray.full((200, c), 0x12345678)
    hip.select_segments(d_q, 200, 128, d_c, c, min_seg, bf, 0, out)
    hip.synchronize()
    assert np.array_equal(out.numpy(), want)
    assert ((want != INV).sum(1) >= min(min_seg, c)).all()


@pytest.mark.parametrize("top_k,beam", [(10, 64), (40, 128), (100, 256), (10, 320), (64, 448), (128, 512)])
def test_search_over_partitions_bit_exact(hip, large_index, top_k, beam):
    from glide_amd.datasets import recall
    from oracle import oracle as O
    L = large_index
    nq = L["queries"].shape[0]
    sp = O.search_params(beam, 32)
    seg_ids = O.select_segments(L["queries"], L["cent"], 2, 1.1)
    e_ids, e_d = np.full((nq, top_k), INV, np.uint32), np.full((nq, top_k), np.finfo(np.float32).max, np.float32)
    d_q, d_seg = hip.DeviceArray.from_numpy(L["queries"]), hip.DeviceArray.from_numpy(seg_ids)
    g_ids, g_d = hip.DeviceArray.from_numpy(e_ids), hip.DeviceArray.from_numpy(e_d)
    for s, seg in enumerate(L["segs"]):
        O.search_sub(seg["data"], seg["graph"], seg["map"], L["queries"], seg_ids, s, int(L["start_points"][s]), top_k, sp, e_ids, e_d)
        d_data, d_graph, d_map = hip.DeviceArray.from_numpy(seg["data"]), hip.DeviceArray.from_numpy(seg["graph"]), hip.DeviceArray.from_numpy(seg["map"])
        hip.search_sub(d_data, 128, d_graph, 32, d_map, d_q, nq, d_seg, 3, s, int(L["start_points"][s]), top_k, sp["beam"],
                       sp["max_iterations"], sp["min_iterations"], sp["hash_bit"], sp["hash_reset_interval"], 0, g_ids, g_d)
        hip.synchronize()
        assert np.array_equal(g_ids.numpy(), e_ids), s
        assert np.array_equal(g_d.numpy(), e_d), s
    gt, _ = O.bruteforce_knn(L["data"], L["queries"], 10)
    assert recall(e_ids[:, :10], gt, 10) >= 0.9          # two partitions per query
    # the same through the grouped form: each partition launches only the queries that selected it
    c = 3
    counts, offsets, lists = hip.DeviceArray(c, np.uint32), hip.DeviceArray(c + 1, np.uint32), hip.DeviceArray(nq * c, np.uint32)
    hip.group_queries(d_seg, nq, c, counts, offsets, lists)
    h_counts, h_off, h_lists = counts.numpy(), offsets.numpy(), lists.numpy()
    assert np.array_equal(h_counts, [(seg_ids == s).sum() for s in range(c)]) and np.array_equal(h_off, np.concatenate([[0], np.cumsum(h_counts)]))
    for s in range(c):
        assert np.array_equal(np.sort(h_lists[h_off[s]:h_off[s + 1]]), np.flatnonzero((seg_ids == s).any(axis=1)))
    l_ids = hip.DeviceArray.from_numpy(np.full((nq, top_k), INV, np.uint32))
    l_d = hip.DeviceArray.from_numpy(np.full((nq, top_k), np.finfo(np.float32).max, np.float32))
    for s, seg in enumerate(L["segs"]):
        d_data, d_graph, d_map = hip.DeviceArray.from_numpy(seg["data"]), hip.DeviceArray.from_numpy(seg["graph"]), hip.DeviceArray.from_numpy(seg["map"])
        hip.search_sub_listed(d_data, 128, d_graph, 32, d_map, d_q, nq, lists.ptr + 4 * int(h_off[s]), int(h_counts[s]), s, int(L["start_points"][s]),
                              top_k, sp["beam"], sp["max_iterations"], sp["min_iterations"], sp["hash_bit"], sp["hash_reset_interval"], 0, l_ids, l_d)
        hip.synchronize()
    assert np.array_equal(l_ids.numpy(), e_ids) and np.array_equal(l_d.numpy(), e_d)
    # and in three launches over the resident index: one wavefront per (query, partition) pair, heads merged per query
    all_data = np.concatenate([seg["data"] for seg in L["segs"]])
    all_graph = np.concatenate([seg["graph"] for seg in L["segs"]])
    all_map = np.concatenate([seg["map"] for seg in L["segs"]])
    lens = np.array([seg["data"].shape[0] for seg in L["segs"]], np.uint32)
    seg_starts = np.concatenate([[0], np.cumsum(lens)[:-1]]).astype(np.uint32)
    p_ids, p_d = hip.DeviceArray((nq, top_k), np.uint32), hip.DeviceArray((nq, top_k), np.float32)
    cnt = hip.new_counters()
    hip.search_partitions(hip.DeviceArray.from_numpy(all_data), 128, hip.DeviceArray.from_numpy(all_graph), 32, hip.DeviceArray.from_numpy(all_map),
                          hip.DeviceArray.from_numpy(seg_starts), hip.DeviceArray.from_numpy(L["start_points"].astype(np.uint32)), c, d_q, nq, d_seg,
                          top_k, sp["beam"], sp["max_iterations"], sp["min_iterations"], sp["hash_bit"], sp["hash_reset_interval"], 0, p_ids, p_d, cnt)
    assert np.array_equal(p_ids.numpy(), e_ids) and np.array_equal(p_d.numpy(), e_d)
    assert hip.read_counters(cnt)[0] > 0


def test_place_and_merge_boundary_bit_exact(hip):
    """The two passes of the merged large build against the oracle's row merge, on rows that take both of its
    branches (at least half of the copy's neighbours already present / fewer) and on rows with empty slots."""
    from oracle import oracle as O
    INV = 0xFFFFFFFF
    rng = np.random.default_rng(5)
    for D in (32, 40, 64, 160):
        n, copies, start = 500, 180, 1000
        local = rng.integers(0, n, (n, D)).astype(np.uint32)
        local[rng.random(local.shape) < 0.2] = INV
        merged = hip.DeviceArray.full((start + n, D), 7)
        hip.place_segment_graph(hip.DeviceArray.from_numpy(local), n, D, start, merged)
        hip.synchronize()
        got = merged.numpy()
        assert (got[:start] == 7).all()
        assert np.array_equal(got[start:], np.where(local == INV, INV, local + np.uint32(start)))

        home = rng.permutation(n)[:copies].astype(np.uint32)
        base = rng.integers(0, n, (n, D)).astype(np.uint32)
        fill = rng.integers(D // 2, D + 1, n)                       # rows as pruning leaves them: filled from the front
        base[np.arange(D)[None, :] >= fill[:, None]] = INV
        bgraph = rng.integers(0, copies, (copies, D)).astype(np.uint32)
        bgraph[rng.random(bgraph.shape) < 0.3] = INV
        for i in range(0, copies, 3):       # many neighbours already in the row: the fill-the-holes branch
            row = base[home[i]]
            k = int(D * 0.7)
            present = np.flatnonzero(np.isin(home, row[row != INV]))
            if present.size:
                bgraph[i, :k] = rng.choice(present, k).astype(np.uint32)
        expect = base.copy()
        branches = set()
        for i in range(copies):
            nb = bgraph[i]
            dup = sum(1 for l in nb[nb != INV] if home[l] in expect[home[i]][:fill[home[i]]])
            branches.add(bool(dup >= D // 2))
            expect[home[i]] = O.merge_boundary_row(expect[home[i]], nb, home)
        assert branches == {True, False}
        d_base = hip.DeviceArray.from_numpy(base)
        hip.merge_boundary_graph(hip.DeviceArray.from_numpy(bgraph), copies, D, hip.DeviceArray.from_numpy(home), d_base)
        hip.synchronize()
        assert np.array_equal(d_base.numpy(), expect), D


def test_search_merged_ranks_every_centroid(hip):
    """glide_hip_search_merged picks the entry among all centroids; glide_hip_search keeps the reference's bucket rule
    (first 64 centroids of a degree-32 index).  Expected results: the oracle's search started from the exact nearest
    centroid of each query."""
    from oracle import oracle as O
    rng = np.random.default_rng(9)
    n, dim, deg, c, nq = 4000, 64, 32, 100, 120
    data = np.rint(rng.random((n, dim)) * 9).astype(np.float32)
    queries = np.rint(rng.random((nq, dim)) * 9).astype(np.float32)
    graph = rng.integers(0, n, (n, deg)).astype(np.uint32)
    centroids = data[rng.permutation(n)[:c]].copy()
    start_points = rng.integers(0, n, c).astype(np.uint32)
    sp = O.search_params(64, deg)
    d2 = ((queries[:, None, :] - centroids[None, :, :]) ** 2).sum(-1)     # small integers: exact in float32
    order = np.lexsort((np.arange(c)[None, :].repeat(nq, 0), d2), axis=1)
    nearest = order[:, 0]
    unique_min = np.sort(d2, axis=1)[:, 0] != np.sort(d2, axis=1)[:, 1]
    assert (nearest >= 64).any() and unique_min.sum() > nq // 2
    e_ids = np.empty((nq, 10), np.uint32)
    for q in range(nq):
        ids, _, _ = O.search(data, graph, centroids[nearest[q]:nearest[q] + 1], start_points[nearest[q]:nearest[q] + 1], queries[q:q + 1], 10, **sp)
        e_ids[q] = ids[0]
    dev = lambda a, t: hip.DeviceArray.from_numpy(a, t)
    ids, dists = hip.DeviceArray((nq, 10), np.uint32), hip.DeviceArray((nq, 10), np.float32)
    args = (dev(data, np.float32), n, dim, dev(graph, np.uint32), deg, dev(centroids, np.float32), c, dev(start_points, np.uint32),
            dev(queries, np.float32), nq, 10, sp["beam"], sp["max_iterations"], sp["min_iterations"], sp["hash_bit"], sp["hash_reset_interval"], 0)
    hip.search_merged(*args, ids, dists)
    hip.synchronize()
    assert np.array_equal(ids.numpy()[unique_min], e_ids[unique_min])
    hip.search(*args, ids, dists)
    hip.synchronize()
    o_ids, _, _ = O.search(data, graph, centroids, start_points, queries, 10, **sp)
    assert np.array_equal(ids.numpy(), o_ids)
    assert (ids.numpy() != e_ids).any()
