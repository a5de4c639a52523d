"""Sub-graph build, reverse edges and refinement of one partition over a seeded sweep of shapes (dimension, kNN
degree, graph degree, build and refine beams incl. the two-half networks, both metrics): bit-exact against the CPU
oracle on small-integer data."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
INV = 0xFFFFFFFF


def _cases():
    rng = np.random.default_rng(777)
    dims = [4, 36, 128, 132, 256, 512, 960, 1536, 2048, 3072, 4096]
    degrees = [8, 24, 32, 64, 96, 160]
    beams = [32, 64, 128, 256, 320, 448, 512]
    out = []
    for i in range(28):
        out.append((i, int(rng.choice(dims)), int(rng.choice(degrees)), int(rng.choice(degrees)), int(rng.choice(beams)), int(rng.choice(beams)),
                    int(rng.integers(0, 2))))
    return out


@pytest.mark.parametrize("case,dim,knn_degree,graph_degree,build_beam,refine_beam,metric", _cases())
def test_segment_build_sweep(case, dim, knn_degree, graph_degree, build_beam, refine_beam, metric):
    from glide_amd import capi as hip
    from oracle import oracle as O
    hip.set_device(0)
    rng = np.random.default_rng(3000 + case)
    n = 500
    hi = 4 if dim >= 512 else 8
    data = rng.integers(0, hi, (n, dim)).astype(np.float32)
    kk = min(knn_degree, n - 1)
    ids, _ = O.bruteforce_knn(data, data, kk, metric, exclude_self=True)
    knn = np.full((n, knn_degree), INV, np.uint32)
    knn[:, :kk] = ids
    knn[rng.random(knn.shape) < 0.05] = INV           # a few holes, as a ragged kNN graph has
    start = int(rng.integers(0, n))
    # The visited table is sized for the rows the search expands: kNN rows in the build, graph rows in the refinement.  (A
    # table that overflows fills in arrival order, which differs between 64 concurrent lanes and a sequential loop.)
    sp_b, sp_r = O.search_params(build_beam, knn_degree), O.search_params(refine_beam, max(knn_degree, graph_degree))
    print("case", case, dict(dim=dim, knn=knn_degree, degree=graph_degree, build_beam=build_beam, refine_beam=refine_beam, metric=metric), flush=True)
    e_built, st = O.build_segment(data, knn, start, graph_degree, sp_b, 1.05, metric)
    e_rev = O.reverse_edges(e_built)
    e_ref, _ = O.refine_segment(data, e_rev, start, sp_r, 1.05, metric)

    d_data, d_knn = hip.DeviceArray.from_numpy(data), hip.DeviceArray.from_numpy(knn)
    g = hip.DeviceArray.full((n, graph_degree), 0xDEADBEEF)
    cnt = hip.new_counters()
    hip.build_segment(d_data, n, dim, d_knn, knn_degree, start, graph_degree, sp_b["beam"], sp_b["max_iterations"], sp_b["min_iterations"],
                      sp_b["hash_bit"], sp_b["hash_reset_interval"], 1.05, metric, g, cnt)
    hip.synchronize()
    assert np.array_equal(g.numpy(), e_built)
    assert hip.read_counters(cnt) == [st["iterations"], st["rows_scored"], st["graph_rows"]]
    rev, rc = hip.DeviceArray((n, graph_degree), np.uint32), hip.DeviceArray(n, np.uint32)
    wb = hip.reverse_edges_workspace_bytes(n, graph_degree)
    hip.reverse_edges(g, n, graph_degree, rev, rc, hip.DeviceArray(wb // 8 + 1, np.uint64), wb)
    hip.insert_reverse(g, rev, rc, n, graph_degree)
    hip.synchronize()
    assert np.array_equal(g.numpy(), e_rev)
    out = hip.DeviceArray.full((n, graph_degree), 0xDEADBEEF)
    hip.refine_segment(d_data, n, dim, g, out, graph_degree, start, sp_r["beam"], sp_r["max_iterations"], sp_r["min_iterations"], sp_r["hash_bit"],
                       sp_r["hash_reset_interval"], 1.05, metric)
    hip.synchronize()
    assert np.array_equal(out.numpy(), e_ref)
