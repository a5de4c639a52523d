"""glide_hip_partition_assign_fixed (the entry point that allocates nothing) against glide_hip_partition_assign.

Two calls in a row share the library's scratch array, the second one smaller, so stale histograms of the first call
would show up in the second one's slots and lengths.  Results are integers and fp32 distances from the same kernels:
they must be identical bit for bit.
"""
import numpy as np
import pytest

from conftest import lowdim_data

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from glide_amd import capi
    capi.set_device(0)
    return capi


def assign_both(hip, data, centroids, bf, metric=0):
    n, dim = data.shape
    c = centroids.shape[0]
    d_data, d_cent = hip.DeviceArray.from_numpy(data, np.float32), hip.DeviceArray.from_numpy(centroids, np.float32)
    out = []
    for fixed in (False, True):
        # outputs start from a pattern no correct call leaves behind
        seg_idx = hip.DeviceArray.from_numpy(np.full((n, 3), 0xDEADBEEF, np.uint32))
        seg_len = hip.DeviceArray.from_numpy(np.full(c + 1, 0xDEADBEEF, np.uint32))
        nearest = hip.DeviceArray.from_numpy(np.full((n, 2), -1.0, np.float32))
        if fixed:
            hip.partition_assign_fixed(d_data, n, dim, d_cent, c, bf, metric, seg_idx, seg_len, nearest)
        else:
            wb = hip.partition_assign_workspace_bytes(n, c)
            ws = hip.DeviceArray(wb // 4 + 1, np.uint32)
            hip.partition_assign(d_data, n, dim, d_cent, c, bf, metric, seg_idx, seg_len, nearest, ws, wb)
        hip.synchronize()
        out.append((seg_idx.numpy(), seg_len.numpy(), nearest.numpy()))
    return out


@pytest.mark.parametrize("shapes", [
    # (points, dim, centroids): first call, then a smaller one on the same scratch
    [(65536, 128, 256), (9000, 128, 16)],
    [(20000, 96, 40), (777, 64, 3)],
    [(5000, 128, 16), (130, 960, 256)],
])
def test_fixed_scratch_matches_workspace_form(hip, shapes):
    from oracle import oracle as O
    assert hip.partition_assign_fixed_max_points() == 65536
    for n, dim, c in shapes:
        print("case", n, dim, c, flush=True)
        data = lowdim_data(n, dim, seed=n + c)
        centroids = O.kmeans(data[:: max(1, n // 2000)], c, iterations=3)
        (w_idx, w_len, w_near), (f_idx, f_len, f_near) = assign_both(hip, data, centroids, 1.04)
        assert np.array_equal(f_len, w_len)
        assert np.array_equal(f_idx, w_idx)
        assert np.array_equal(f_near.view(np.uint32), w_near.view(np.uint32))
        assert int(f_len[:c].sum()) == n


def test_fixed_scratch_rejects_oversize_and_bad_arguments(hip):
    n, dim, c = 65537, 8, 2
    d_data = hip.DeviceArray((n, dim), np.float32)
    d_cent = hip.DeviceArray((c, dim), np.float32)
    seg_idx, seg_len = hip.DeviceArray((n, 3), np.uint32), hip.DeviceArray(c + 1, np.uint32)
    rc = hip.partition_assign_fixed(d_data, n, dim, d_cent, c, 1.04, 0, seg_idx, seg_len, None, check_status=False)
    assert rc == -1   # GLIDE_ERR_UNSUPPORTED: more points than the scratch array holds
    assert "supported" in hip.error_string(rc)
    rc = hip.partition_assign_fixed(d_data, 100, dim, d_cent, 300, 1.04, 0, seg_idx, seg_len, None, check_status=False)
    assert rc == -1   # more than 256 centroids, as the workspace form
    rc = hip.partition_assign_fixed(None, 100, dim, d_cent, c, 1.04, 0, seg_idx, seg_len, None, check_status=False)
    assert rc == -2
    # an empty batch only clears the lengths
    seg_len.upload(np.full(c + 1, 7, np.uint32))
    hip.partition_assign_fixed(d_data, 0, dim, d_cent, c, 1.04, 0, seg_idx, seg_len, None)
    hip.synchronize()
    assert np.array_equal(seg_len.numpy(), np.zeros(c + 1, np.uint32))


def test_fixed_scratch_calls_allocate_nothing(hip):
    """What the entry point is for: once its first call on the device has looked up the scratch array, further calls of
    any size leave the device's free memory where it was (every input and output is allocated beforehand)."""
    from oracle import oracle as O
    cases = []
    for n, dim, c in ((4096, 128, 16), (65536, 128, 256), (333, 64, 5), (20000, 96, 40)):
        data = lowdim_data(n, dim, seed=n)
        cent = O.kmeans(data[:: max(1, n // 1000)], c, iterations=2)
        cases.append((n, dim, c, hip.DeviceArray.from_numpy(data), hip.DeviceArray.from_numpy(cent), hip.DeviceArray((n, 3), np.uint32),
                      hip.DeviceArray(c + 1, np.uint32), hip.DeviceArray((n, 2), np.float32)))
    n, dim, c, d_data, d_cent, seg_idx, seg_len, nearest = cases[0]
    hip.partition_assign_fixed(d_data, n, dim, d_cent, c, 1.04, 0, seg_idx, seg_len, nearest)      # first call: symbol lookup
    hip.synchronize()
    free_before, total = hip.mem_info()
    assert 0 < free_before <= total
    for _ in range(3):
        for n, dim, c, d_data, d_cent, seg_idx, seg_len, nearest in cases:
            print("fixed call", n, dim, c, flush=True)
            hip.partition_assign_fixed(d_data, n, dim, d_cent, c, 1.04, 0, seg_idx, seg_len, nearest)
            assert hip.mem_info()[0] == free_before, "a call changed the device's free memory while it was in flight"
    hip.synchronize()
    assert hip.mem_info()[0] == free_before
    # the workspace form needs memory the caller brings: the same figure moves when that workspace is allocated
    wb = hip.partition_assign_workspace_bytes(65536, 256)
    ws = hip.DeviceArray(max(wb // 4 + 1, 1 << 20), np.uint32)
    assert hip.mem_info()[0] < free_before
    ws.free()
