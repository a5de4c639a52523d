"""GPU graph construction (sub-graph build, boundary merge, reverse edges, refine) against the CPU oracle."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
INV = 0xFFFFFFFF


@pytest.fixture(scope="module")
def hip():
    from glide_amd import capi
    capi.set_device(0)
    return capi


@pytest.fixture(scope="module")
def stages(small_index):
    """Oracle outputs after every stage, from the same partitioning / kNN graph."""
    from oracle import oracle as O
    idx = small_index
    n, D, K = idx["data"].shape[0], 32, 32
    c = idx["centroids"].shape[0]
    sp = O.search_params(64, K)
    g_sub, st_sub = O.build_subgraph(idx["reorder_data"], n, idx["knn"], idx["map"], idx["seg_start"], idx["seg_len"],
                                     idx["local_start_points"], D, sp, 1.05)
    g_bnd, st_bnd = O.build_boundary(idx["reorder_data"], n, idx["knn"], idx["map"], int(idx["local_start_points"][c]),
                                     g_sub.copy(), sp, 1.05)
    g_rev = O.reverse_edges(g_bnd)
    sp_ref = O.search_params(128, K)
    g_ref, st_ref = O.refine(idx["data"], g_rev, idx["centroids"], idx["start_points"], sp_ref, 1.05)
    return dict(sp=sp, sp_ref=sp_ref, sub=g_sub, st_sub=st_sub, bnd=g_bnd, st_bnd=st_bnd, rev=g_rev, ref=g_ref, st_ref=st_ref)


def dev(hip, idx):
    return dict(rdata=hip.DeviceArray.from_numpy(idx["reorder_data"], np.float32), knn=hip.DeviceArray.from_numpy(idx["knn"], np.uint32),
                map=hip.DeviceArray.from_numpy(idx["map"], np.uint32), ss=hip.DeviceArray.from_numpy(idx["seg_start"], np.uint32),
                sl=hip.DeviceArray.from_numpy(idx["seg_len"], np.uint32), lsp=hip.DeviceArray.from_numpy(idx["local_start_points"], np.uint32))


def gpu_build_sub(hip, idx, sp, D=32, relaxant=1.05, metric=0):
    d = dev(hip, idx)
    n, dim = idx["data"].shape
    graph = hip.DeviceArray.full((n, D), INV)
    cnt = hip.new_counters()
    hip.build_subgraph(d["rdata"], n, dim, d["knn"], idx["knn"].shape[1], d["map"], d["ss"], d["sl"], idx["seg_start"].size, d["lsp"],
                       D, sp["beam"], sp["max_iterations"], sp["min_iterations"], sp["hash_bit"], sp["hash_reset_interval"],
                       relaxant, metric, graph, cnt)
    hip.synchronize()
    return d, graph, cnt


def test_build_subgraph_bit_exact(hip, small_index, stages):
    _, graph, cnt = gpu_build_sub(hip, small_index, stages["sp"])
    assert np.array_equal(graph.numpy(), stages["sub"])
    st = stages["st_sub"]
    assert hip.read_counters(cnt) == [st["iterations"], st["rows_scored"], st["graph_rows"]]


def test_build_boundary_bit_exact(hip, small_index, stages):
    idx, sp = small_index, stages["sp"]
    d, graph, _ = gpu_build_sub(hip, idx, sp)
    n, dim = idx["data"].shape
    c = idx["centroids"].shape[0]
    rn = idx["reorder_data"].shape[0]
    assert rn > n, "fixture must have boundary points"
    hip.build_boundary(d["rdata"], n, rn, dim, d["knn"], 32, d["map"], int(idx["local_start_points"][c]), 32, sp["beam"],
                       sp["max_iterations"], sp["min_iterations"], sp["hash_bit"], sp["hash_reset_interval"], 1.05, 0, graph)
    hip.synchronize()
    got = graph.numpy()
    assert np.array_equal(got, stages["bnd"])
    assert (got != stages["sub"]).any(), "the merge must change some rows"


def gpu_reverse(hip, graph_np):
    n, D = graph_np.shape
    g = hip.DeviceArray.from_numpy(graph_np, np.uint32)
    rev, cnt = hip.DeviceArray((n, D), np.uint32), hip.DeviceArray(n, np.uint32)
    wb = hip.reverse_edges_workspace_bytes(n, D)
    ws = hip.DeviceArray(wb // 8 + 1, np.uint64)
    hip.reverse_edges(g, n, D, rev, cnt, ws, wb)
    hip.insert_reverse(g, rev, cnt, n, D)
    hip.synchronize()
    return g.numpy(), rev.numpy(), cnt.numpy()


def test_reverse_edges_bit_exact_and_invariants(hip, stages):
    before = stages["bnd"]
    got, rev, cnt = gpu_reverse(hip, before)
    assert np.array_equal(got, stages["rev"])
    n, D = before.shape
    # invariants that hold for any arrival order: only empty slots change; each inserted u in row v had v in row u
    changed = got != before
    assert (before[changed] == INV).all()
    rows, cols = np.nonzero(changed)
    for v, c in list(zip(rows, cols))[:2000]:
        u = got[v, c]
        assert v in before[u] and u not in before[v]
    assert (np.minimum(cnt, D) == (rev != INV).sum(1)).all()


def test_reverse_edges_hub_and_degree64(hip):
    # a hub that everybody points at (bucket far larger than a wavefront) and a wider graph
    rng = np.random.default_rng(3)
    from oracle import oracle as O
    n, D = 3000, 64
    g = rng.integers(0, n, (n, D)).astype(np.uint32)
    g[:, 0] = 7                       # hub
    g[rng.random((n, D)) < 0.4] = INV
    g[7] = INV                        # the hub's row is empty: it takes the first D sources in (column, source) order
    got, rev, cnt = gpu_reverse(hip, g)
    assert np.array_equal(got, O.reverse_edges(g))
    assert cnt[7] >= n * 0.5


def test_refine_bit_exact(hip, small_index, stages):
    idx, sp = small_index, stages["sp_ref"]
    n, dim = idx["data"].shape
    g_in = hip.DeviceArray.from_numpy(stages["rev"], np.uint32)
    g_out = hip.DeviceArray.full((n, 32), 0xDEADBEEF)
    data = hip.DeviceArray.from_numpy(idx["data"], np.float32)
    cent = hip.DeviceArray.from_numpy(idx["centroids"], np.float32)
    spd = hip.DeviceArray.from_numpy(idx["start_points"], np.uint32)
    cntd = hip.new_counters()
    assert (stages["rev"] == INV).any(), "fixture must leave holes for refinement"
    hip.refine(data, n, dim, g_in, g_out, 32, cent, idx["centroids"].shape[0], spd, sp["beam"], sp["max_iterations"],
               sp["min_iterations"], sp["hash_bit"], sp["hash_reset_interval"], 1.05, 0, cntd)
    hip.synchronize()
    assert np.array_equal(g_out.numpy(), stages["ref"])
    st = stages["st_ref"]
    assert hip.read_counters(cntd) == [st["iterations"], st["rows_scored"], st["graph_rows"]]
    assert np.array_equal(g_in.numpy(), stages["rev"])      # input untouched
    # the processing order (here: partition order, as the host layer passes it) does not change the result
    g_out2 = hip.DeviceArray.full((n, 32), 0xDEADBEEF)
    order = hip.DeviceArray.from_numpy(idx["map"][:n].astype(np.uint32))
    assert np.array_equal(np.sort(idx["map"][:n]), np.arange(n))
    hip.refine(data, n, dim, g_in, g_out2, 32, cent, idx["centroids"].shape[0], spd, sp["beam"], sp["max_iterations"],
               sp["min_iterations"], sp["hash_bit"], sp["hash_reset_interval"], 1.05, 0, order=order)
    hip.synchronize()
    assert np.array_equal(g_out2.numpy(), stages["ref"])


def test_built_graph_is_searchable(hip, small_index, stages):
    from glide_amd.datasets import recall
    from oracle import oracle as O
    from test_gpu_search import run_gpu_search
    idx = small_index
    gt, _ = O.bruteforce_knn(idx["data"], idx["queries"], 10)
    sp = O.search_params(64, 32)
    ids, _, _ = run_gpu_search(hip, idx["data"], stages["ref"], idx["centroids"], idx["start_points"], idx["queries"], 10, sp)
    assert recall(ids, gt, 10) >= 0.95


def test_wide_degree_and_beam_bit_exact(hip):
    """Degree 160 with beams 320 (build) and 512 (refine): the candidate sort and the beam merge both run as two
    half-wave networks (reference search_kernel.cuh:38-94, :149-232) and the prune tables hold up to 256 entries."""
    from conftest import lowdim_data
    from oracle import oracle as O
    K = D = 160
    n, c = 2500, 2
    data = lowdim_data(n, 64, seed=11)
    idx = O.build_index(data, c, graph_degree=32, knn_degree=32, nnd_iterations=2, refine_beam=0)
    rdata = idx["reorder_data"]
    rn = rdata.shape[0]
    assert rn > n
    knn = np.full((rn, K), INV, np.uint32)                     # exact neighbours inside each partition
    for s, l in zip(idx["seg_start"].tolist(), idx["seg_len"].tolist()):
        ids, _ = O.bruteforce_knn(rdata[s:s + l], rdata[s:s + l], min(K, l - 1), 0, exclude_self=True)
        knn[s:s + l, :ids.shape[1]] = ids
    idx = dict(idx, knn=knn, data=data)
    sp = O.search_params(320, K)
    e_sub, st_sub = O.build_subgraph(rdata, n, knn, idx["map"], idx["seg_start"], idx["seg_len"], idx["local_start_points"], D, sp, 1.05)
    e_bnd, _ = O.build_boundary(rdata, n, knn, idx["map"], int(idx["local_start_points"][c]), e_sub.copy(), sp, 1.05)
    e_rev = O.reverse_edges(e_bnd)
    sp_ref = O.search_params(512, K)
    e_ref, st_ref = O.refine(data, e_rev, idx["centroids"], idx["start_points"], sp_ref, 1.05)

    print("wide build", sp, flush=True)
    d, graph, cnt = gpu_build_sub(hip, idx, sp, D=D)
    assert np.array_equal(graph.numpy(), e_sub)
    assert hip.read_counters(cnt) == [st_sub["iterations"], st_sub["rows_scored"], st_sub["graph_rows"]]
    print("wide boundary", flush=True)
    hip.build_boundary(d["rdata"], n, rn, 64, d["knn"], K, d["map"], int(idx["local_start_points"][c]), D, sp["beam"],
                       sp["max_iterations"], sp["min_iterations"], sp["hash_bit"], sp["hash_reset_interval"], 1.05, 0, graph)
    hip.synchronize()
    assert np.array_equal(graph.numpy(), e_bnd)
    print("wide reverse", flush=True)
    assert np.array_equal(gpu_reverse(hip, e_bnd)[0], e_rev)
    print("wide refine", sp_ref, flush=True)
    g_in = hip.DeviceArray.from_numpy(e_rev, np.uint32)
    g_out = hip.DeviceArray.full((n, D), 0xDEADBEEF)
    cntd = hip.new_counters()
    hip.refine(hip.DeviceArray.from_numpy(data, np.float32), n, 64, g_in, g_out, D, hip.DeviceArray.from_numpy(idx["centroids"], np.float32), c,
               hip.DeviceArray.from_numpy(idx["start_points"], np.uint32), sp_ref["beam"], sp_ref["max_iterations"], sp_ref["min_iterations"],
               sp_ref["hash_bit"], sp_ref["hash_reset_interval"], 1.05, 0, cntd)
    hip.synchronize()
    assert np.array_equal(g_out.numpy(), e_ref)
    assert hip.read_counters(cntd) == [st_ref["iterations"], st_ref["rows_scored"], st_ref["graph_rows"]]
