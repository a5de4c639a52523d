"""Degenerate partitionings through every stage: an empty partition, partitions of one and of five points (fewer
points than list slots), no boundary points at all, and a boundary list.  Each GPU stage against the CPU oracle on the
same inputs; the kNN graph comes from the GPU (NN-descent is not reproducible bit for bit), everything after it is."""
import numpy as np
import pytest

from conftest import lowdim_data

pytestmark = pytest.mark.gpu
INV = 0xFFFFFFFF


@pytest.mark.parametrize("boundary_factor", [0.0, 1.1])
def test_degenerate_partitions_through_every_stage(boundary_factor):
    from glide_amd import capi as hip
    from oracle import oracle as O
    from test_gpu_nnd import gpu_nnd
    from test_gpu_search import run_gpu_search
    hip.set_device(0)
    dim, D, K = 32, 32, 32
    body = lowdim_data(900, dim, seed=71)
    lone = np.full((1, dim), 250.0, np.float32)                          # a partition of one point
    few = np.full((5, dim), 5.0, np.float32) + np.arange(5, dtype=np.float32)[:, None]   # a partition of five
    data = np.concatenate([body, lone, few]).astype(np.float32)
    n = data.shape[0]
    centroids = np.concatenate([O.kmeans(body, 2, 10, 3), lone, few.mean(0, keepdims=True), np.full((1, dim), -4000.0, np.float32)]).astype(np.float32)
    c = centroids.shape[0]                                                # the last centroid attracts nothing

    # ---- partition + reorder
    e_idx, e_len, near = O.partition_assign(data, centroids, boundary_factor)
    d_data, d_cent = hip.DeviceArray.from_numpy(data), hip.DeviceArray.from_numpy(centroids)
    d_idx, d_len = hip.DeviceArray((n, 3), np.uint32), hip.DeviceArray(c + 1, np.uint32)
    wb = hip.partition_assign_workspace_bytes(n, c)
    ws = hip.DeviceArray(wb // 4 + 1, np.uint32)
    hip.partition_assign(d_data, n, dim, d_cent, c, boundary_factor, 0, d_idx, d_len, None, ws, wb)
    hip.synchronize()
    seg_len = d_len.numpy()
    assert np.array_equal(seg_len, e_len) and np.array_equal(d_idx.numpy(), e_idx)
    assert seg_len[4] == 0 and seg_len[2] == 1 and seg_len[3] == 5 and seg_len[0] > 400 and seg_len[1] > 400
    assert (seg_len[c] > 0) == (boundary_factor > 0)
    starts = O.segment_starts(seg_len)
    rn = n + int(seg_len[c])
    e_rdata, e_map = O.reorder(data, e_idx, starts, rn)
    d_re, d_map = hip.DeviceArray((rn, dim), np.float32), hip.DeviceArray(rn, np.uint32)
    hip.reorder(d_data, n, dim, d_idx, hip.DeviceArray.from_numpy(starts), d_re, d_map)
    hip.synchronize()
    assert np.array_equal(d_re.numpy(), e_rdata) and np.array_equal(d_map.numpy(), e_map)

    # ---- kNN graph: ids stay inside their partition, also where a partition has fewer points than list slots
    knn, _ = gpu_nnd(hip, e_rdata, starts[:c + 1], seg_len, K, 6)
    for s, l in zip(starts[:c + 1].tolist(), seg_len.tolist()):
        assert (knn[s:s + l] < max(l, 1)).all()
    s0, l0 = int(starts[0]), int(seg_len[0])
    gt, _ = O.bruteforce_knn(e_rdata[s0:s0 + l0], e_rdata[s0:s0 + 100], K, exclude_self=True)
    from glide_amd.datasets import recall
    assert recall(knn[s0:s0 + 100], gt, K) >= 0.9

    # ---- sub-graphs, boundary merge, reverse edges, refine, search: bit-exact
    local_sp = np.array([min(3, max(int(l), 1) - 1) for l in seg_len], np.uint32)
    start_points = np.array([e_map[starts[i] + local_sp[i]] if seg_len[i] else 0 for i in range(c)], np.uint32)
    sp = O.search_params(64, K)
    e_graph, _ = O.build_subgraph(e_rdata, n, knn, e_map, starts[:c + 1], seg_len, local_sp, D, sp, 1.05)
    d_knn = hip.DeviceArray.from_numpy(knn)
    graph = hip.DeviceArray.full((n, D), INV)
    hip.build_subgraph(d_re, n, dim, d_knn, K, d_map, hip.DeviceArray.from_numpy(starts[:c + 1].astype(np.uint32)), hip.DeviceArray.from_numpy(seg_len),
                       c + 1, hip.DeviceArray.from_numpy(local_sp), D, sp["beam"], sp["max_iterations"], sp["min_iterations"], sp["hash_bit"],
                       sp["hash_reset_interval"], 1.05, 0, graph, None)
    hip.synchronize()
    assert np.array_equal(graph.numpy(), e_graph)
    if rn > n:
        e_graph, _ = O.build_boundary(e_rdata, n, knn, e_map, int(local_sp[c]), e_graph, sp, 1.05)
        hip.build_boundary(d_re, n, rn, dim, d_knn, K, d_map, int(local_sp[c]), D, sp["beam"], sp["max_iterations"], sp["min_iterations"],
                           sp["hash_bit"], sp["hash_reset_interval"], 1.05, 0, graph)
        hip.synchronize()
        assert np.array_equal(graph.numpy(), e_graph)
    e_rev = O.reverse_edges(e_graph)
    rev, cnt = hip.DeviceArray((n, D), np.uint32), hip.DeviceArray(n, np.uint32)
    wb = hip.reverse_edges_workspace_bytes(n, D)
    hip.reverse_edges(graph, n, D, rev, cnt, hip.DeviceArray(wb // 8 + 1, np.uint64), wb)
    hip.insert_reverse(graph, rev, cnt, n, D)
    hip.synchronize()
    assert np.array_equal(graph.numpy(), e_rev)
    sp_r = O.search_params(128, K)
    e_ref, _ = O.refine(data, e_rev, centroids, start_points, sp_r, 1.05)
    out = hip.DeviceArray.full((n, D), 0xDEADBEEF)
    hip.refine(d_data, n, dim, graph, out, D, d_cent, c, hip.DeviceArray.from_numpy(start_points), sp_r["beam"], sp_r["max_iterations"],
               sp_r["min_iterations"], sp_r["hash_bit"], sp_r["hash_reset_interval"], 1.05, 0)
    hip.synchronize()
    assert np.array_equal(out.numpy(), e_ref)
    queries = np.concatenate([lowdim_data(50, dim, seed=72), lone, few[:2], np.full((1, dim), -3900.0, np.float32)]).astype(np.float32)
    ssp = O.search_params(64, D)
    e_ids, e_d, _ = O.search(data, e_ref, centroids, start_points, queries, 10, **ssp)
    g_ids, g_d, _ = run_gpu_search(hip, data, e_ref, centroids, start_points, queries, 10, ssp)
    assert np.array_equal(g_ids, e_ids) and np.array_equal(g_d, e_d)


def test_empty_inputs_are_no_ops():
    """No points / no queries: every stage returns without touching its outputs (the partition stage reports zero
    lengths), as a loop over nothing would; sentinels in the output buffers stay where they are."""
    from glide_amd import capi as hip
    from oracle import oracle as O
    hip.set_device(0)
    dim, c, D, K = 32, 3, 16, 16
    buf = lambda shape, dtype=np.uint32: hip.DeviceArray.full(shape, 7, dtype)
    d_rows, d_cent = hip.DeviceArray.from_numpy(lowdim_data(64, dim, seed=1)), hip.DeviceArray.from_numpy(lowdim_data(c, dim, seed=2))
    sp = O.search_params(64, K)
    beam_args = (sp["beam"], sp["max_iterations"], sp["min_iterations"], sp["hash_bit"], sp["hash_reset_interval"])

    d_idx, d_len = buf((8, 3)), buf(c + 1)
    wb = hip.partition_assign_workspace_bytes(8, c)
    ws = hip.DeviceArray(wb // 4 + 1, np.uint32)
    hip.partition_assign(d_rows, 0, dim, d_cent, c, 1.04, 0, d_idx, d_len, None, ws, wb)
    hip.synchronize()
    assert not d_len.numpy().any() and (d_idx.numpy() == 7).all()

    d_re, d_map, d_starts = buf((8, dim), np.float32), buf(8), hip.DeviceArray.from_numpy(np.zeros(c + 1, np.uint32))
    hip.reorder(d_rows, 0, dim, d_idx, d_starts, d_re, d_map)
    hip.sample_rows(d_rows, dim, d_map, 0, d_re)

    d_knn, d_graph, d_out, d_cnt, d_sp = buf((8, K)), buf((8, D)), buf((8, D)), buf(8), hip.DeviceArray.from_numpy(np.zeros(c + 1, np.uint32))
    hip.build_subgraph(d_rows, 0, dim, d_knn, K, d_map, d_starts, d_starts, c + 1, d_sp, D, *beam_args, 1.05, 0, d_graph, None)
    wb = hip.reverse_edges_workspace_bytes(8, D)
    hip.reverse_edges(d_graph, 0, D, d_out, d_cnt, hip.DeviceArray(wb // 8 + 1, np.uint64), wb)
    hip.insert_reverse(d_graph, d_out, d_cnt, 0, D)
    hip.refine(d_rows, 0, dim, d_graph, d_out, D, d_cent, c, d_sp, *beam_args, 1.05, 0)
    d_ids = buf((4, c))
    hip.select_segments(d_rows, 0, dim, d_cent, c, 2, 1.1, 0, d_ids)
    res_i, res_d = buf((4, 10)), buf((4, 10), np.float32)
    hip.search(d_rows, 64, dim, d_graph, D, d_cent, c, d_sp, d_rows, 0, 10, *beam_args, 0, res_i, res_d)
    hip.synchronize()
    for d in (d_re, d_map, d_graph, d_out, d_cnt, d_ids, res_i, res_d):
        assert (d.numpy() == 7).all()
