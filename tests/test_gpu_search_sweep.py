"""Beam search over a seeded sweep of shapes (dimension buckets, degree buckets, beam buckets incl. the two-half
networks, top-k, centroid counts, both metrics): ids, distances and counters bit-exact against the CPU oracle on
small-integer data, where every distance is exact in float32."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _cases():
    rng = np.random.default_rng(20240)
    dims = [4, 8, 36, 100, 128, 132, 256, 260, 512, 960, 1024, 1028, 1536, 2048, 2052, 3072, 4096]
    degrees = [8, 16, 24, 32, 40, 64, 72, 96, 128, 160, 256]
    beams = [32, 64, 96, 128, 192, 256, 288, 320, 448, 480, 512]
    out = []
    for i in range(72):
        dim, deg, beam = int(rng.choice(dims)), int(rng.choice(degrees)), int(rng.choice(beams))
        top_k = int(rng.integers(1, min(beam, 128) + 1))
        cents = int(rng.choice([1, 2, 7, 32, 33, 64, 100, 200]))
        out.append((i, dim, deg, beam, top_k, cents, int(rng.integers(0, 2))))
    return out


@pytest.mark.parametrize("case,dim,deg,beam,top_k,cents,metric", _cases())
def test_search_sweep(case, dim, deg, beam, top_k, cents, metric):
    from glide_amd import capi as hip
    from oracle import oracle as O
    from test_gpu_search import run_gpu_search
    hip.set_device(0)
    rng = np.random.default_rng(1000 + case)
    n, nq = 1200, 16
    hi = 4 if dim >= 512 else 8                      # sums stay below 2^24
    data = rng.integers(0, hi, (n, dim)).astype(np.float32)
    queries = rng.integers(0, hi, (nq, dim)).astype(np.float32)
    if metric == O.COSINE:                            # cosine is squared L2 of the rows as given: keep integers
        pass
    graph = rng.integers(0, n, (n, deg)).astype(np.uint32)
    graph[rng.random(graph.shape) < 0.15] = 0xFFFFFFFF
    centroids = data[rng.permutation(n)[:cents]].copy()
    start_points = rng.integers(0, n, cents).astype(np.uint32)
    sp = O.search_params(beam, deg)
    print("case", case, dict(dim=dim, degree=deg, beam=beam, top_k=top_k, centroids=cents, metric=metric), sp, flush=True)
    args = (data, graph, centroids, start_points, queries, top_k)
    e_ids, e_d, st = O.search(*args, metric=metric, **sp)
    g_ids, g_d, cnt = run_gpu_search(hip, *args, sp, metric=metric, counters=True)
    assert np.array_equal(g_ids, e_ids) and np.array_equal(g_d, e_d)
    assert cnt == [st["iterations"], st["rows_scored"], st["graph_rows"]]
