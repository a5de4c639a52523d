"""GPU beam search against the CPU oracle on the same index, through the C ABI."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from glide_amd import capi
    capi.set_device(0)
    return capi


def run_gpu_search(hip, data, graph, centroids, start_points, queries, top_k, sp, metric=0, counters=False):
    d = dict(data=hip.DeviceArray.from_numpy(data, np.float32), graph=hip.DeviceArray.from_numpy(graph, np.uint32),
             cent=hip.DeviceArray.from_numpy(centroids, np.float32), sp=hip.DeviceArray.from_numpy(start_points, np.uint32),
             q=hip.DeviceArray.from_numpy(queries, np.float32))
    nq = queries.shape[0]
    ids, dists = hip.DeviceArray((nq, top_k), np.uint32), hip.DeviceArray((nq, top_k), np.float32)
    cnt = hip.new_counters() if counters else None
    hip.search(d["data"], data.shape[0], data.shape[1], d["graph"], graph.shape[1], d["cent"], centroids.shape[0], d["sp"],
               d["q"], nq, top_k, sp["beam"], sp["max_iterations"], sp["min_iterations"], sp["hash_bit"],
               sp["hash_reset_interval"], metric, ids, dists, cnt)
    hip.synchronize()
    return ids.numpy(), dists.numpy(), (hip.read_counters(cnt) if counters else None)


@pytest.mark.parametrize("beam,top_k", [(32, 10), (64, 10), (96, 32), (128, 10), (256, 100), (288, 10), (384, 100), (512, 10)])
def test_search_bit_exact_on_integer_data(hip, small_index, beam, top_k):
    from oracle import oracle as O
    idx = small_index
    sp = O.search_params(beam, 32)
    eids, edists, est = O.search(idx["data"], idx["graph"], idx["centroids"], idx["start_points"], idx["queries"], top_k, **sp)
    gids, gdists, gcnt = run_gpu_search(hip, idx["data"], idx["graph"], idx["centroids"], idx["start_points"],
                                        idx["queries"], top_k, sp, counters=True)
    assert np.array_equal(gids, eids)
    assert np.array_equal(gdists, edists)
    assert gcnt == [est["iterations"], est["rows_scored"], est["graph_rows"]]


def test_search_recall_against_brute_force(hip, small_index):
    from glide_amd.datasets import recall
    from oracle import oracle as O
    idx = small_index
    gt, _ = O.bruteforce_knn(idx["data"], idx["queries"], 10)
    sp = O.search_params(64, 32)
    gids, _, _ = run_gpu_search(hip, idx["data"], idx["graph"], idx["centroids"], idx["start_points"], idx["queries"], 10, sp)
    assert recall(gids, gt, 10) >= 0.95


def test_search_graph_with_holes_and_min_iterations(hip, small_index):
    from oracle import oracle as O
    idx = small_index
    graph = idx["graph"].copy()
    rng = np.random.default_rng(0)
    graph[rng.random(graph.shape) < 0.3] = 0xFFFFFFFF          # empty slots anywhere in a row
    graph[5] = 0xFFFFFFFF                                      # a node without neighbours
    sp = O.search_params(64, 32)
    sp["min_iterations"] = 40
    args = (idx["data"], graph, idx["centroids"], idx["start_points"], idx["queries"], 10)
    eids, edists, _ = O.search(*args, **sp)
    gids, gdists, _ = run_gpu_search(hip, *args, sp)
    assert np.array_equal(gids, eids) and np.array_equal(gdists, edists)


def test_search_cosine_float_data(hip):
    from oracle import oracle as O
    from conftest import lowdim_float_data
    data = lowdim_float_data(4000, 96, seed=3)
    queries = lowdim_float_data(200, 96, seed=4)
    idx = O.build_index(data, 2, graph_degree=32, knn_degree=32, nnd_iterations=6, metric=O.COSINE)
    sp = O.search_params(64, 32)
    args = (data, idx["graph"], idx["centroids"], idx["start_points"], queries, 10)
    eids, edists, _ = O.search(*args, metric=O.COSINE, **sp)
    gids, gdists, _ = run_gpu_search(hip, *args, sp, metric=O.COSINE)
    # float data: the 64-lane reduction order differs from the 32-lane one, so distances agree to 1e-5 relative
    # and an id may differ only where two candidates are closer than that
    same = (gids == eids).mean()
    assert same >= 0.99, same
    assert np.allclose(gdists[gids == eids], edists[gids == eids], rtol=1e-5, atol=1e-7)


def test_search_degree64_dim960(hip):
    from oracle import oracle as O
    rng = np.random.default_rng(7)
    n, dim, deg = 1500, 960, 64
    data = np.rint(rng.random((n, dim)) * 15).astype(np.float32)      # small integers: exact sums
    queries = np.rint(rng.random((40, dim)) * 15).astype(np.float32)
    graph = rng.integers(0, n, (n, deg)).astype(np.uint32)
    centroids = data[:40].copy()                                        # > 32 centroids: the 64-wide centroid network
    start_points = rng.integers(0, n, 40).astype(np.uint32)
    for beam in (64, 128):
        sp = O.search_params(beam, deg)
        args = (data, graph, centroids, start_points, queries, 10)
        eids, edists, _ = O.search(*args, **sp)
        gids, gdists, _ = run_gpu_search(hip, *args, sp)
        assert np.array_equal(gids, eids) and np.array_equal(gdists, edists)


@pytest.mark.parametrize("dim,deg", [(960, 64), (384, 32), (1024, 160), (1536, 32), (2048, 64), (3072, 32), (4096, 64)])
def test_long_rows_small_and_large_batches_agree(hip, dim, deg):
    """Rows of more than 256 dims are searched by a team of four wavefronts per query while the batch is small and by one
    wavefront per query once it fills the chip; both forms must give the oracle's ids, distances and counters (integer
    data: exact sums, frequent ties), for every beam bucket including the two-half merge above 256, and a query must get
    the same answer whichever batch it arrives in."""
    from oracle import oracle as O
    rng = np.random.default_rng(dim + deg)
    n, big = 2500, 2100                         # 2100 queries: beyond two wavefronts per SIMD for a team of four
    data = np.rint(rng.random((n, dim)) * 9).astype(np.float32)
    queries = np.rint(rng.random((big, dim)) * 9).astype(np.float32)
    graph = rng.integers(0, n, (n, deg)).astype(np.uint32)
    graph[rng.random(graph.shape) < 0.05] = 0xFFFFFFFF
    centroids = data[:5].copy()
    start_points = rng.integers(0, n, 5).astype(np.uint32)
    for beam in (32, 128, 256, 448):
        sp = O.search_params(beam, deg)
        print("dim", dim, "degree", deg, "beam", beam, flush=True)
        small = run_gpu_search(hip, data, graph, centroids, start_points, queries[:70], 10, sp, counters=True)
        eids, edists, est = O.search(data, graph, centroids, start_points, queries[:70], 10, **sp)
        assert np.array_equal(small[0], eids) and np.array_equal(small[1], edists)
        assert small[2] == [est["iterations"], est["rows_scored"], est["graph_rows"]]
        large = run_gpu_search(hip, data, graph, centroids, start_points, queries, 10, sp, counters=True)
        assert np.array_equal(large[0][:70], eids) and np.array_equal(large[1][:70], edists)
        pick = rng.choice(big, 40, replace=False)
        eids, edists, _ = O.search(data, graph, centroids, start_points, queries[pick], 10, **sp)
        assert np.array_equal(large[0][pick], eids) and np.array_equal(large[1][pick], edists)
        one = run_gpu_search(hip, data, graph, centroids, start_points, queries[pick[:1]], 10, sp)
        assert np.array_equal(one[0], eids[:1]) and np.array_equal(one[1], edists[:1])


@pytest.mark.parametrize("deg", [32, 64])
def test_wide_beams_on_distinct_keys(hip, deg):
    """Beams above 256 on keys that are all distinct, and on keys that repeat.  Points on a line and queries beyond its
    ends make all distances of a search distinct (and exact); a second data set repeats every position once, so that
    beams hold equal keys, where the order the reference's two-half merge leaves is the network's own.  Beams 288 and 448
    run the merge with its lane permutations, beam 512 the whole-beam form; ids, distances and counters must be the
    oracle's."""
    from oracle import oracle as O
    rng = np.random.default_rng(deg)
    n = 3000
    for repeats in (1, 2):
        data = np.zeros((n, 4), np.float32)
        data[:, 0] = rng.permutation(n) // repeats
        queries = np.zeros((120, 4), np.float32)
        queries[:60, 0] = n + 0.5 + np.arange(60)
        queries[60:, 0] = -0.5 - np.arange(60)
        graph = rng.integers(0, n, (n, deg)).astype(np.uint32)
        graph[rng.random(graph.shape) < 0.1] = 0xFFFFFFFF
        centroids = data[:3].copy()
        start_points = rng.integers(0, n, 3).astype(np.uint32)
        for beam in (288, 448, 512):
            sp = O.search_params(beam, deg)
            args = (data, graph, centroids, start_points, queries, 10)
            eids, edists, est = O.search(*args, **sp)
            print("degree", deg, "repeats", repeats, "beam", beam, flush=True)
            gids, gdists, gcnt = run_gpu_search(hip, *args, sp, counters=True)
            assert np.array_equal(gids, eids) and np.array_equal(gdists, edists)
            assert gcnt == [est["iterations"], est["rows_scored"], est["graph_rows"]]
            if repeats == 1:
                assert np.unique(edists[0]).size == 10


@pytest.mark.parametrize("deg", [160, 256])
def test_search_degree_above_128(hip, deg):
    """Degrees above 128 sort the candidate list as two half-wave networks, beams above 256 merge the same way
    (reference search_kernel.cuh:38-94 and :149-232); integer data, so ties between distinct ids are frequent."""
    from oracle import oracle as O
    rng = np.random.default_rng(deg)
    n, dim = 3000, 64
    data = np.rint(rng.random((n, dim)) * 7).astype(np.float32)
    queries = np.rint(rng.random((60, dim)) * 7).astype(np.float32)
    graph = rng.integers(0, n, (n, deg)).astype(np.uint32)
    graph[rng.random(graph.shape) < 0.1] = 0xFFFFFFFF
    centroids = data[:8].copy()
    start_points = rng.integers(0, n, 8).astype(np.uint32)
    for beam in (64, 256, 320, 512):
        sp = O.search_params(beam, deg)
        args = (data, graph, centroids, start_points, queries, 10)
        eids, edists, est = O.search(*args, **sp)
        print("degree", deg, "beam", beam, sp, flush=True)
        gids, gdists, gcnt = run_gpu_search(hip, *args, sp, counters=True)
        assert np.array_equal(gids, eids) and np.array_equal(gdists, edists)
        assert gcnt == [est["iterations"], est["rows_scored"], est["graph_rows"]]


def test_search_rejects_unsupported_sizes(hip):
    d = hip.DeviceArray(4096, np.float32)
    base = dict(data=d, num=8, dim=128, graph=d, graph_degree=32, centroids=d, centroid_num=2, start_points=d, queries=d,
                query_num=1, top_k=10, beam=64, max_iterations=10, min_iterations=0, hash_bit=8, hash_reset_interval=2,
                metric=0, result_ids=d, result_dists=d)
    for key, bad in (("beam", 544), ("beam", 300), ("graph_degree", 257), ("centroid_num", 300), ("dim", 130), ("dim", 4100), ("top_k", 65)):
        with pytest.raises(hip.GlideHipError) as e:
            hip.search(**{**base, key: bad})
        assert e.value.code == -1, key
    hip.search(**{**base, "query_num": 0})   # empty batch is a no-op
