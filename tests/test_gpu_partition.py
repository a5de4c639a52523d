"""GPU locality partitioning (assignment, slots, reorder, sampling, k-means) against the CPU oracle."""
import numpy as np
import pytest

from conftest import lowdim_data, lowdim_float_data

pytestmark = pytest.mark.gpu
INV = 0xFFFFFFFF


@pytest.fixture(scope="module")
def hip():
    from glide_amd import capi
    capi.set_device(0)
    return capi


def gpu_assign(hip, data, centroids, bf, metric=0):
    n, dim = data.shape
    c = centroids.shape[0]
    d_data, d_cent = hip.DeviceArray.from_numpy(data, np.float32), hip.DeviceArray.from_numpy(centroids, np.float32)
    seg_idx, seg_len = hip.DeviceArray((n, 3), np.uint32), hip.DeviceArray(c + 1, np.uint32)
    nearest = hip.DeviceArray((n, 2), np.float32)
    wb = hip.partition_assign_workspace_bytes(n, c)
    ws = hip.DeviceArray(wb // 4 + 1, np.uint32)
    hip.partition_assign(d_data, n, dim, d_cent, c, bf, metric, seg_idx, seg_len, nearest, ws, wb)
    hip.synchronize()
    return d_data, seg_idx, seg_len.numpy(), nearest.numpy()


@pytest.mark.parametrize("n,dim,c,metric", [(5000, 128, 16, 0), (3001, 96, 5, 1), (2000, 128, 1, 0), (4000, 64, 40, 0),
                                            (3000, 128, 100, 0), (2500, 32, 200, 0), (1500, 960, 16, 0), (100, 128, 3, 0),
                                            (1000, 4, 7, 0), (1200, 36, 33, 0), (900, 1024, 256, 0), (700, 132, 64, 1),
                                            # at most 32 centroids of at most 128 dims: the kernel that keeps the centroids in LDS
                                            (2222, 100, 32, 0), (1800, 64, 31, 0), (1300, 36, 2, 1), (4100, 124, 17, 0),
                                            (800, 4096, 24, 0), (600, 3072, 40, 1)])
def test_assign_matches_oracle(hip, n, dim, c, metric):
    from oracle import oracle as O
    data = lowdim_float_data(n, dim, seed=n) if metric == 1 else lowdim_data(n, dim, seed=n)
    centroids = O.kmeans(data[:: max(1, n // 2000)], c, iterations=5)
    bf = 1.04
    e_idx, e_len, e_near = O.partition_assign(data, centroids, bf, metric)
    _, seg_idx, g_len, g_near = gpu_assign(hip, data, centroids, bf, metric)
    g_idx = seg_idx.numpy()
    # distances: 64-lane vs 32-lane summation order
    assert np.allclose(g_near[:, 0], e_near[:, 0], rtol=1e-5)
    if c > 1:
        assert np.allclose(g_near[:, 1], e_near[:, 1], rtol=1e-5)
    # decisions may differ only where the reference's own inputs are within rounding of a tie / of the threshold
    ratio = e_near[:, 1] / e_near[:, 0] if c > 1 else np.full(n, np.inf)
    safe_seg = (np.abs(ratio - 1.0) > 1e-4) if c > 1 else np.ones(n, bool)
    safe_bnd = np.abs(ratio - bf) > 1e-4
    assert np.array_equal(g_idx[safe_seg, 0], e_idx[safe_seg, 0])
    assert np.array_equal((g_idx[:, 2] != INV)[safe_bnd & safe_seg], (e_idx[:, 2] != INV)[safe_bnd & safe_seg])
    assert safe_seg.mean() > 0.99 and safe_bnd.mean() > 0.99
    # slot numbering: point order within each segment, lengths add up
    assert g_len[:c].sum() == n
    for s in range(c):
        members = np.nonzero(g_idx[:, 0] == s)[0]
        assert np.array_equal(g_idx[members, 1], np.arange(members.size))
        assert g_len[s] == members.size
    bmem = np.nonzero(g_idx[:, 2] != INV)[0]
    assert np.array_equal(g_idx[bmem, 2], np.arange(bmem.size)) and g_len[c] == bmem.size
    if safe_seg.all() and safe_bnd.all():
        assert np.array_equal(g_idx, e_idx) and np.array_equal(g_len, e_len)


@pytest.mark.parametrize("n,dim,c,copies", [(1500, 128, 48, 12), (600, 64, 200, 200), (500, 256, 40, 9), (700, 128, 256, 6)])
def test_assign_coincident_centroids(hip, n, dim, c, copies):
    """Centroids that coincide: more candidates tie for the two nearest than the ranking pass hands on per lane, so the
    points near them are measured against every centroid.  Integer rows make every distance exact: the two nearest
    distances and the boundary flags must be the oracle's to the bit.  Between centroids at exactly the same distance
    the reference's choice falls out of its bitonic network; here the smaller centroid id wins."""
    from oracle import oracle as O
    data = lowdim_data(n, dim, seed=n + c)
    centroids = O.kmeans(data, c, iterations=3)
    centroids = np.round(centroids).astype(np.float32)
    rng = np.random.default_rng(c)
    where = rng.permutation(c)[:copies]
    centroids[where] = centroids[where[0]]
    e_idx, e_len, e_near = O.partition_assign(data, centroids, 1.04, 0)
    _, seg_idx, g_len, g_near = gpu_assign(hip, data, centroids, 1.04, 0)
    g_idx = seg_idx.numpy()
    assert np.array_equal(g_near, e_near)
    assert np.array_equal(g_idx[:, 2], e_idx[:, 2]) and g_len[c] == e_len[c]
    tied = e_near[:, 0] == e_near[:, 1]
    assert np.array_equal(g_idx[~tied, 0], e_idx[~tied, 0])
    assert tied.sum() > 0
    for p in np.nonzero(tied)[0]:
        d = np.sqrt(((data[p] - centroids) ** 2).sum(1, dtype=np.float32))
        assert g_idx[p, 0] == np.nonzero(d == d.min())[0][0], p
    assert (g_idx[tied, 0] == where.min()).any()
    for s_ in range(c):
        members = np.nonzero(g_idx[:, 0] == s_)[0]
        assert np.array_equal(g_idx[members, 1], np.arange(members.size)) and g_len[s_] == members.size


def test_assign_brute_force_float64(hip):
    # independent of the oracle: float64 argmin and ratio with a margin
    rng = np.random.default_rng(0)
    data = lowdim_data(4000, 128, seed=9)
    centroids = data[rng.permutation(4000)[:24]] + rng.standard_normal((24, 128)).astype(np.float32)
    _, seg_idx, g_len, _ = gpu_assign(hip, data, centroids, 1.1)
    g = seg_idx.numpy()
    d = np.sqrt(((data[:, None, :].astype(np.float64) - centroids[None].astype(np.float64)) ** 2).sum(-1))
    order = np.argsort(d, axis=1)
    d0, d1 = d[np.arange(4000), order[:, 0]], d[np.arange(4000), order[:, 1]]
    clear = (d1 / d0 - 1) > 1e-4
    assert np.array_equal(g[clear, 0], order[clear, 0])
    far = np.abs(d1 / d0 - 1.1) > 1e-4
    assert np.array_equal((g[:, 2] != INV)[far & clear], (d1 / d0 <= 1.1)[far & clear])


def test_reorder_matches_oracle(hip):
    from oracle import oracle as O
    data = lowdim_data(3000, 128, seed=4)
    centroids = O.kmeans(data, 6, iterations=5)
    d_data, seg_idx, seg_len, _ = gpu_assign(hip, data, centroids, 1.04)
    starts = O.segment_starts(seg_len)
    rn = 3000 + int(seg_len[6])
    d_starts = hip.DeviceArray.from_numpy(starts, np.uint32)
    rdata, mp = hip.DeviceArray((rn, 128), np.float32), hip.DeviceArray(rn, np.uint32)
    hip.reorder(d_data, 3000, 128, seg_idx, d_starts, rdata, mp)
    hip.synchronize()
    e_rdata, e_map = O.reorder(data, seg_idx.numpy(), starts, rn)
    assert np.array_equal(mp.numpy(), e_map)
    assert np.array_equal(rdata.numpy(), e_rdata)
    assert np.array_equal(data[mp.numpy()], rdata.numpy())          # every reorder row is its original
    assert sorted(mp.numpy()[:3000].tolist()) == list(range(3000))  # the first num rows are a permutation


def test_sample_rows_and_kmeans(hip):
    from oracle import oracle as O
    rng = np.random.default_rng(2)
    data = lowdim_data(6000, 128, seed=5)
    ids = rng.permutation(6000)[:1500].astype(np.uint32)
    d_data, d_ids = hip.DeviceArray.from_numpy(data), hip.DeviceArray.from_numpy(ids)
    sample = hip.DeviceArray((1500, 128), np.float32)
    hip.sample_rows(d_data, 128, d_ids, 1500, sample)
    hip.synchronize()
    assert np.array_equal(sample.numpy(), data[ids])
    # Lloyd from the same initial centroids: same assignments as a float64 Lloyd => centroids agree to rounding
    k = 8
    init = data[ids[:k]].copy()
    cent = hip.DeviceArray.from_numpy(init)
    wb = hip.kmeans_workspace_bytes(k, 128)
    ws = hip.DeviceArray(wb // 4 + 1, np.uint32)
    hip.kmeans_fit(sample, 1500, 128, k, 10, cent, ws, wb)
    hip.synchronize()
    ref = init.astype(np.float64)
    x = data[ids].astype(np.float64)
    for _ in range(10):
        a = ((x[:, None] - ref[None]) ** 2).sum(-1).argmin(1)
        for c in range(k):
            if (a == c).any():
                ref[c] = x[a == c].mean(0)
    got = cent.numpy()
    assert np.allclose(got, ref, rtol=1e-4, atol=1e-2)
    inertia = lambda c: ((x[:, None] - c[None]) ** 2).sum(-1).min(1).sum()
    assert inertia(got.astype(np.float64)) <= inertia(init.astype(np.float64))
