"""Points whose length is no multiple of four values.  The reference's kernels loop over single values and take any
dim (distance.cuh:9-27); here rows are read in 16-byte pieces, so such points are held with zeros behind them
(glide_hip_copy_rows, index.pad_rows).  A zero coordinate changes no distance, so every stage must equal the CPU
oracle's on the points as they are, bit for bit on integer-valued data."""
import numpy as np
import pytest

from conftest import lowdim_data

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from glide_amd import capi
    capi.set_device(0)
    return capi


@pytest.mark.parametrize("src_dim,dst_dim", [(50, 52), (52, 50), (25, 28), (1, 4), (7, 7), (129, 132)])
def test_copy_rows(hip, src_dim, dst_dim):
    num = 1237
    src = np.random.default_rng(src_dim).standard_normal((num, src_dim)).astype(np.float32)
    d_src = hip.DeviceArray.from_numpy(src)
    d_dst = hip.DeviceArray.full((num, dst_dim), 7.0, np.float32)
    hip.copy_rows(d_src, num, src_dim, d_dst, dst_dim)
    hip.synchronize()
    keep = min(src_dim, dst_dim)
    want = np.zeros((num, dst_dim), np.float32)
    want[:, :keep] = src[:, :keep]
    assert np.array_equal(d_dst.numpy(), want)
    hip.copy_rows(d_src, 0, src_dim, d_dst, dst_dim)      # no rows: nothing launched


@pytest.mark.parametrize("dim", [25, 50, 101, 3070])      # 3070: held as 3072, the row shape with a whole wavefront per row
def test_pipeline_on_rows_of_any_length(hip, dim):
    from glide_amd import datasets as D, index as G
    from oracle import oracle as O
    num, nq, parts, degree = (6000, 200, 3, 32) if dim < 1024 else (3000, 100, 3, 32)
    data, queries = lowdim_data(num, dim, seed=71), lowdim_data(nq, dim, seed=72)
    if dim > 1024:      # values 0..8, so that sums of 3070 squared differences stay exact in float32
        data, queries = np.rint(data / 32), np.rint(queries / 32)
    print("dim", dim, flush=True)
    held = (dim + 3) // 4 * 4

    pp = G.PartitionParameter(centroid_num=parts, boundary_factor=1.04, sample_factor=0.05, metric=0)
    d_re, d_map, h_start, h_len, d_cent = G.preprocess(pp, hip.DeviceArray.from_numpy(data))
    assert d_re.shape[1] == held and d_cent.shape[1] == held
    assert not d_re.numpy()[:, dim:].any() and not d_cent.numpy()[:, dim:].any()       # the padding stays zero
    centroids, rdata, h_map = G.cut_rows(d_cent, dim), G.cut_rows(d_re, dim), d_map.numpy()
    assert centroids.shape == (parts, dim) and np.array_equal(rdata, data[h_map])
    seg_idx, seg_len, near = O.partition_assign(data, centroids, 1.04, 0)
    ratio = near[:, 1] / near[:, 0]
    if (np.abs(ratio - 1.04) > 1e-4).all() and (np.abs(ratio - 1) > 1e-4).all():       # centroids are not integer-valued
        assert np.array_equal(seg_len, h_len)
        _, map_cpu = O.reorder(data, seg_idx, O.segment_starts(seg_len), num + int(seg_len[parts]))
        assert np.array_equal(map_cpu, h_map)

    d_knn = G.build_nnd(G.NNDescentParameter(graph_degree=32, max_iterations=8, seed=0, termination_threshold=0.0), d_re, h_start, h_len)
    knn = d_knn.numpy()
    s, l = int(h_start[0]), int(h_len[0])
    gt, _ = O.bruteforce_knn(rdata[s:s + l], rdata[s:s + 200], 32, exclude_self=True)
    assert D.recall(knn[s:s + 200], gt, 32) >= (0.95 if dim < 1024 else 0.8)      # coarse values: many equal distances

    index = G.GLIDE(degree, data, centroids, 0)              # points and centroids in their own length: held padded
    assert index.dim() == held
    bp = G.IndexParameter(graph_degree=degree, knn_degree=32, relaxant_factor=1.05)
    local_sp, start_points = index.start_point_select(h_start, h_len, h_map, bp.seed)
    index.build(bp, G.make_search_parameter(64, 32), G.make_search_parameter(128, 32), d_knn, h_start, h_len, d_map, d_re)
    graph = index.d_graph.numpy()

    # the oracle on the points as they are, from the same kNN graph and entry points: the same graph
    ps = O.search_params(64, 32)
    g, _ = O.build_subgraph(rdata, num, knn, h_map, h_start, h_len, local_sp, degree, ps, 1.05, 0)
    if rdata.shape[0] > num:
        g, _ = O.build_boundary(rdata, num, knn, h_map, int(local_sp[parts]), g, ps, 1.05, 0)
    g = O.reverse_edges(g)
    g, _ = O.refine(data, g, centroids, start_points, O.search_params(128, 32), 1.05, 0)
    assert np.array_equal(g, graph)

    # ... and the same search results, for queries handed over in their own length
    for beam in (32, 128, 320):
        sp = G.make_search_parameter(beam, degree, 10)
        ids, dists = index.search(sp, hip.DeviceArray.from_numpy(queries))
        e_ids, e_dists, _ = O.search(data, graph, centroids, start_points, queries, 10, sp.beam, sp.max_iterations, sp.min_iterations,
                                     sp.hash_bit, sp.hash_reset_interval, 0)
        assert np.array_equal(ids, e_ids) and np.array_equal(dists, e_dists), beam
    truth, _ = O.bruteforce_knn(data, queries, 10)
    assert D.recall(ids, truth, 10) >= (0.95 if dim < 1024 else 0.8)
    with pytest.raises(ValueError):
        index.search(sp, hip.DeviceArray.from_numpy(queries[:, :dim - 4]))
