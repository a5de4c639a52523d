"""The 1M-point configurations at their real size: 16 partitions, top-10; graph degree 32 and 10 000 queries for 128 dims
Euclidean on the benchmark's mixture and on data of low intrinsic dimension and for 96 dims cosine on the normalised
mixture; graph degree 64, kNN degree 64 and 1 000 queries for the 960-dim configuration.

What the CPU oracle can finish in seconds at this size is compared bit for bit (the sub-graph rows of the first
points, searches of a sample of the queries on the finished index); everything else is held to properties that do
not depend on the size: the partition is a partition, reordered rows are the rows they claim to be, every list of
the kNN graph is a set of local ids without the node itself, graph rows hold distinct ids, a second build from the
same kNN graph gives the same graph, results are sorted, distinct, carry the exact distance of the id they name and
do not depend on how the queries are ordered or batched.  On the float data a reassociated sum can flip a near-tie,
so "bit for bit" becomes "all but a few rows" there and distances are compared to 1e-5.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

N, C = 1_000_000, 16
# name: generator, dims, metric, integer-valued (sums exact in fp32), graph degree, kNN degree, queries, graph recall@32 expected
CONFIGS = {"lowdim_integer": ("lowdim_integer", 128, 0, True, 32, 32, 10_000, 0.95), "gmm_clipped": ("gmm_clipped", 128, 0, True, 32, 32, 10_000, 0.95),
           "gmm_normalized_cosine": ("gmm_normalized", 96, 1, False, 32, 32, 10_000, 0.95),
           # the termination limit of NN-descent grows with the row length (nn_descent.cuh:1280), so the 960-dim build stops
           # after fewer rounds: recall@32 0.89 here, on the GPU and in the CPU restatement alike
           "beta_scaled_960": ("beta_scaled", 960, 0, False, 64, 64, 1_000, 0.85)}
INVALID = 0xFFFFFFFF


@pytest.fixture(scope="module")
def hip():
    from glide_amd import capi
    capi.set_device(0)
    return capi


# the benchmark's mixture (64 far-apart components: search recall is low by construction) and data of low intrinsic
# dimension, on which recall is meaningful
@pytest.fixture(scope="module", params=list(CONFIGS))
def world(hip, request):
    """Data, queries, the partitioning, the kNN graph and the finished index, all made on the GPU."""
    from glide_amd import datasets as Ds, index as G
    gen_name, DIM, metric, exact, D, K, NQ, knn_recall = CONFIGS[request.param]
    gen = getattr(Ds, gen_name)
    data, queries = gen(N, DIM, seed=1234), gen(NQ, DIM, seed=4321)
    print("data", request.param, data.shape, flush=True)
    d_data = hip.DeviceArray.from_numpy(data)
    pp = G.PartitionParameter(centroid_num=C, boundary_factor=1.04, sample_factor=0.01, metric=metric)
    d_re, d_map, h_start, h_len, d_cent = G.preprocess(pp, d_data)
    rdata, h_map, centroids = d_re.numpy(), d_map.numpy(), d_cent.numpy()
    d_knn = G.build_nnd(G.NNDescentParameter(graph_degree=K, max_iterations=20), d_re, h_start, h_len)
    knn = d_knn.numpy()
    print("partitioned and kNN built", rdata.shape, knn.shape, flush=True)
    # a second run from the same input: k-means seeding, Lloyd steps (fixed-point sums) and slot numbering are all
    # independent of the order in which wavefronts run, so centroids, map and segment lengths repeat bit for bit
    d_re2, d_map2, h_start2, h_len2, d_cent2 = G.preprocess(pp, d_data)
    assert np.array_equal(d_cent2.numpy(), centroids) and np.array_equal(d_map2.numpy(), h_map) and np.array_equal(h_len2, h_len)
    for d in (d_re2, d_map2, d_cent2):
        d.free()
    w = dict(kind=request.param, metric=metric, exact=exact, D=D, K=K, NQ=NQ, knn_recall=knn_recall, data=data, queries=queries, rdata=rdata, map=h_map, seg_start=h_start.copy(), seg_len=h_len.copy(), centroids=centroids, knn=knn)

    # the sub-graph stage alone, for the comparison with the oracle
    index = G.GLIDE(D, d_data, d_cent, metric)
    bp = G.IndexParameter(graph_degree=D, knn_degree=K, relaxant_factor=1.05)
    local_sp, start_points = index.start_point_select(h_start, h_len, h_map, bp.seed)
    sp_b = G.make_search_parameter(64, K)
    d_ss, d_sl, d_lsp = (hip.DeviceArray.from_numpy(np.ascontiguousarray(a, dtype=np.uint32)) for a in (h_start, h_len, local_sp))
    d_sub = hip.DeviceArray.full((N, D), INVALID)
    hip.build_subgraph(d_re, N, DIM, d_knn, K, d_map, d_ss, d_sl, C + 1, d_lsp, D, sp_b.beam, sp_b.max_iterations, sp_b.min_iterations,
                       sp_b.hash_bit, sp_b.hash_reset_interval, 1.05, metric, d_sub)
    hip.synchronize()
    w.update(sub=d_sub.numpy(), local_sp=local_sp, start_points=start_points, sp_b=sp_b)
    d_sub.free()

    # two complete builds from the same kNN graph (build() consumes its device inputs, so they are copied first)
    graphs = []
    for _ in range(2):
        idx = G.GLIDE(D, d_data, d_cent, metric)
        idx.build(bp, sp_b, G.make_search_parameter(128, K), hip.DeviceArray.from_numpy(knn), h_start, h_len,
                  hip.DeviceArray.from_numpy(h_map), hip.DeviceArray.from_numpy(rdata))
        graphs.append(idx.d_graph.numpy())
        index = idx
    assert np.array_equal(index.d_start_points.numpy(), start_points)
    w.update(index=index, graph=graphs[1], graph_again=graphs[0], d_queries=hip.DeviceArray.from_numpy(queries))
    print("index built", flush=True)
    return w


def _truth(world):
    if "truth" not in world:
        from oracle import oracle as O
        world["truth"] = O.bruteforce_knn(world["data"], world["queries"][:min(1000, world["NQ"])], 10, world["metric"])[0].astype(np.uint32)
    return world["truth"]


def test_partition_is_a_partition(world):
    seg_start, seg_len, mp, rdata, data = world["seg_start"], world["seg_len"], world["map"], world["rdata"], world["data"]
    assert int(seg_len[:C].sum()) == N
    assert np.array_equal(seg_start[:C + 1], np.concatenate([[0], np.cumsum(seg_len[:C])]).astype(np.uint32))
    nb = int(seg_len[C])
    assert mp.shape[0] == N + nb and rdata.shape[0] == N + nb
    assert np.array_equal(np.sort(mp[:N]), np.arange(N, dtype=np.uint32)), "the first N map entries are a permutation"
    assert np.unique(mp[N:]).size == nb, "a point has at most one boundary copy"
    assert np.array_equal(rdata, data[mp]), "reordered rows are the rows the map names"
    # inside a partition the points keep their original order (slots are numbered in point order)
    for s, l in zip(seg_start[:C].tolist(), seg_len[:C].tolist()):
        assert np.all(np.diff(mp[s:s + l].astype(np.int64)) > 0)
    assert np.all(np.diff(mp[N:].astype(np.int64)) > 0)


def test_partition_assignment_on_a_sample(world):
    data, centroids, mp, seg_start, seg_len = world["data"], world["centroids"], world["map"], world["seg_start"], world["seg_len"]
    owner = np.empty(N, dtype=np.int64)
    for c in range(C):
        owner[mp[seg_start[c]:seg_start[c] + seg_len[c]]] = c
    boundary = np.zeros(N, dtype=bool)
    boundary[mp[N:]] = True
    pick = np.random.default_rng(5).choice(N, 20_000, replace=False)
    d = ((data[pick, None, :].astype(np.float64) - centroids[None].astype(np.float64)) ** 2).sum(-1)
    if world["metric"] == 0:
        d = np.sqrt(d)      # the boundary ratio is one of distances for Euclidean, of squared distances for cosine
    order = np.argsort(d, axis=1)
    d0, d1 = d[np.arange(pick.size), order[:, 0]], d[np.arange(pick.size), order[:, 1]]
    clear = d1 - d0 > 1e-4 * d1          # away from ties between the two nearest centroids
    assert clear.mean() > 0.99
    assert np.array_equal(owner[pick][clear], order[:, 0][clear])
    ratio = d1 / d0
    sure = np.abs(ratio - 1.04) > 1e-4     # away from the boundary threshold
    assert np.array_equal(boundary[pick][sure], (ratio <= 1.04)[sure])


def test_knn_graph_lists(world):
    D, K, NQ = world["D"], world["K"], world["NQ"]
    from glide_amd import datasets as Ds
    from oracle import oracle as O
    knn, seg_start, seg_len, rdata = world["knn"], world["seg_start"], world["seg_len"], world["rdata"]
    assert knn.shape == (rdata.shape[0], K)
    recalls = []
    for s, l in zip(seg_start.tolist(), seg_len.tolist()):
        rows = knn[s:s + l].astype(np.int64)
        assert rows.min() >= 0 and rows.max() < l, "ids are local to the partition"
        assert not (rows == np.arange(l)[:, None]).any(), "no list holds its own node"
        srt = np.sort(rows, axis=1)
        assert (np.diff(srt, axis=1) > 0).all(), "no list holds an id twice"
        m, ke = 100, 32
        ids, _ = O.bruteforce_knn(rdata[s:s + l], rdata[s:s + m], ke + 1, world["metric"])
        truth = np.array([[x for x in ids[i].tolist() if x != i][:ke] for i in range(m)], dtype=np.uint32)
        recalls.append(Ds.recall(knn[s:s + m, :ke], truth, ke))
    print("graph recall@32 per partition", np.round(recalls, 4), flush=True)
    assert np.mean(recalls) >= world["knn_recall"]


def test_subgraph_rows_equal_the_oracle(world):
    """The first points in partition order, searched over their whole partition of the full-size kNN graph."""
    D, K, NQ = world["D"], world["K"], world["NQ"]
    from oracle import oracle as O
    m = 1500 if world["data"].shape[1] <= 128 else 400
    sp = O.search_params(64, K)
    assert (sp["beam"], sp["max_iterations"], sp["hash_bit"]) == (world["sp_b"].beam, world["sp_b"].max_iterations, world["sp_b"].hash_bit)
    expect = np.full((N, D), INVALID, dtype=np.uint32)
    O.build_subgraph(world["rdata"], m, world["knn"], world["map"], world["seg_start"], world["seg_len"], world["local_sp"], D, sp, 1.05,
                     world["metric"], graph=expect)
    rows = world["map"][:m]
    same = (world["sub"][rows] == expect[rows]).all(axis=1).mean()
    print("sub-graph rows identical:", same, flush=True)
    assert same == 1.0 if world["exact"] else same >= 0.97
    assert (expect[rows] != INVALID).any()


def test_graph_rows_and_determinism(world):
    D, K, NQ = world["D"], world["K"], world["NQ"]
    g = world["graph"]
    assert g.shape == (N, D)
    assert np.array_equal(g, world["graph_again"]), "two builds from one kNN graph differ"
    valid = g != INVALID
    assert g[valid].max() < N
    # A row can name its own point only through the reference's entry-point quirk (graph_kernel.cuh:295-298: the entry's
    # neighbour that is excluded is the one whose LOCAL id equals the point's REORDER id), i.e. for kNN neighbours of a
    # partition's entry point; the oracle reproduces it (test_subgraph_rows_equal_the_oracle, test_gpu_graph.py).
    own = int((g == np.arange(N, dtype=np.uint32)[:, None]).any(axis=1).sum())
    print("rows that name their own point:", own, flush=True)
    assert own <= (C + 1) * K
    srt = np.sort(g.astype(np.int64), axis=1)
    dup = (np.diff(srt, axis=1) == 0) & (srt[:, 1:] != INVALID)
    assert not dup.any(), "a row names a point twice"
    assert valid.any(axis=1).all(), "a point without any neighbour"


@pytest.mark.parametrize("beam", [32, 256])
def test_search_sample_equals_the_oracle(hip, world, beam):
    D, K, NQ = world["D"], world["K"], world["NQ"]
    from glide_amd import index as G
    from oracle import oracle as O
    sp = G.make_search_parameter(beam, D, 10)
    ids, dists = world["index"].search(sp, world["d_queries"])
    pick = np.random.default_rng(beam).choice(NQ, 48, replace=False)
    e_ids, e_dists, _ = O.search(world["data"], world["graph"], world["centroids"], world["start_points"], world["queries"][pick], 10,
                                 sp.beam, sp.max_iterations, sp.min_iterations, sp.hash_bit, sp.hash_reset_interval, world["metric"])
    if world["exact"]:
        assert np.array_equal(ids[pick], e_ids)
        assert np.array_equal(dists[pick], e_dists)
    else:
        same = (ids[pick] == e_ids).all(axis=1).mean()
        print("result rows identical:", same, flush=True)
        assert same >= 0.9
        assert np.allclose(dists[pick][:, 0], e_dists[:, 0], rtol=1e-5)


@pytest.mark.parametrize("beam", [32, 64])
def test_search_properties(hip, world, beam):
    D, K, NQ = world["D"], world["K"], world["NQ"]
    from glide_amd import datasets as Ds, index as G
    data, queries = world["data"], world["queries"]
    sp = G.make_search_parameter(beam, D, 10)
    ids, dists = world["index"].search(sp, world["d_queries"])
    assert ids.max() < N, "every query fills its top-10 here"
    assert (np.diff(dists, axis=1) >= 0).all(), "results are sorted by distance"
    assert (np.diff(np.sort(ids.astype(np.int64), axis=1), axis=1) > 0).all(), "a result names a point twice"
    # the distance reported is the distance of the point named: integer data, so the fp32 sum is exact
    sq = ((data[ids.reshape(-1)].astype(np.float64) - np.repeat(queries, 10, axis=0).astype(np.float64)) ** 2).sum(1)
    if world["exact"]:
        assert np.array_equal(dists.reshape(-1), np.sqrt(sq.astype(np.float32)))
    else:
        assert np.allclose(dists.reshape(-1), sq if world["metric"] == 1 else np.sqrt(sq), rtol=1e-5, atol=1e-7)
    # the order and the batching of the queries do not matter
    perm = np.random.default_rng(1).permutation(NQ)
    p_ids, p_dists = world["index"].search(sp, hip.DeviceArray.from_numpy(np.ascontiguousarray(queries[perm])))
    assert np.array_equal(p_ids, ids[perm]) and np.array_equal(p_dists, dists[perm])
    h_ids, _ = world["index"].search(sp, hip.DeviceArray.from_numpy(np.ascontiguousarray(queries[:NQ // 3])))
    assert np.array_equal(h_ids, ids[:NQ // 3])
    # recall against exact neighbours of the first 1000 queries (the oracle's brute force)
    gt = _truth(world)
    r = Ds.recall(ids[:gt.shape[0]], gt, 10)
    print("beam", beam, "recall@10", r, flush=True)
    if world["kind"] == "lowdim_integer":
        assert r >= (0.96 if beam == 32 else 0.99)


def test_recall_is_bounded_by_what_the_entry_point_reaches(hip, world):
    """A search enters through the one start point of the query's nearest centroid (search_kernel.cuh:270-271,
    glide_impl.cuh:43-75) and only scores neighbours of nodes it has scored: a true neighbour that no directed path from
    that start point reaches cannot be returned at any beam.  The bound is computed on the host by breadth-first search
    over the finished 1M x 32 graph; every beam of the reference's range must stay below it query by query, and the widest
    beam must come close to it -- which is what makes the low recall of the mixtures a property of the algorithm on that
    data (components the kNN graph does not connect) and not of this implementation."""
    from glide_amd import datasets as Ds, index as G
    D, K, NQ = world["D"], world["K"], world["NQ"]
    gt = _truth(world)
    m = gt.shape[0]
    bound, reach_frac, per_query = Ds.reachable_recall_bound(world["graph"], world["centroids"], world["start_points"], world["queries"][:m], gt,
                                                             world["metric"])
    print(world["kind"], "reachable bound on recall@10: %.4f; an average start point reaches %.3f of the points" % (bound, reach_frac), flush=True)
    recalls = {}
    for beam in (32, 64, 128, 256, 512):
        sp = G.make_search_parameter(beam, D, 10)
        ids, _ = world["index"].search(sp, world["d_queries"])
        found = np.array([np.isin(ids[q], gt[q]).sum() / 10.0 for q in range(m)])
        assert (found <= per_query + 1e-9).all(), "beam %d returned a true neighbour the entry point cannot reach" % beam
        recalls[beam] = float(found.mean())
    print(world["kind"], "recall@10 by beam", {b: round(r, 4) for b, r in recalls.items()}, flush=True)
    assert all(recalls[a] <= recalls[b] + 0.005 for a, b in zip((32, 64, 128, 256), (64, 128, 256, 512)))
    assert recalls[512] <= bound and bound - recalls[512] <= 0.05
    if world["kind"] == "lowdim_integer":
        assert bound >= 0.999 and recalls[32] >= 0.96
    elif world["kind"] == "beta_scaled_960":
        assert bound >= 0.99 and recalls[512] >= 0.95, "the 960-dim configuration reaches the metric's operating point inside the reference's beam range"
    else:
        assert bound < 0.5, "the mixtures' components are not connected: no beam can reach recall@10 0.95"
