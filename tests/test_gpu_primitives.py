"""GPU parity of the device primitives against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from glide_amd import capi
    capi.set_device(0)
    return capi


@pytest.mark.parametrize("m", [32, 64, 128, 256, 512])
def test_bitonic_sort_bit_exact_with_ties(hip, m):
    from oracle import oracle as O
    rng = np.random.default_rng(m)
    batch = 64
    keys = rng.integers(0, 12, (batch, m)).astype(np.float32)     # many equal keys
    keys[: batch // 2] = rng.standard_normal((batch // 2, m)).astype(np.float32)
    keys[0] = 3.0                                                   # all equal
    keys[1, ::2] = np.float32(3.4e38)
    vals = rng.permutation(batch * m).reshape(batch, m).astype(np.uint32)
    dk, dv = hip.DeviceArray.from_numpy(keys), hip.DeviceArray.from_numpy(vals)
    hip.bitonic_sort_kv(dk, dv, m, batch)
    gk, gv = dk.numpy(), dv.numpy()
    for b in range(batch):
        ek, ev = O.bitonic_warp_sort(keys[b], vals[b])
        assert np.array_equal(gk[b], ek), (m, b)
        assert np.array_equal(gv[b], ev), (m, b)


@pytest.mark.parametrize("m", [64, 128, 256, 512])
def test_bitonic_merge_bit_exact(hip, m):
    from oracle import oracle as O
    rng = np.random.default_rng(100 + m)
    batch = 32
    keys = np.empty((batch, m), np.float32)
    for b in range(batch):
        up = np.sort(rng.integers(0, 40, m // 2)).astype(np.float32)
        down = np.sort(rng.integers(0, 40, m // 2))[::-1].astype(np.float32)
        keys[b] = np.concatenate([up, down])
    keys[0] = rng.integers(0, 9, m)  # not bitonic at all: the network is still a fixed function of its input
    vals = rng.permutation(batch * m).reshape(batch, m).astype(np.uint32)
    dk, dv = hip.DeviceArray.from_numpy(keys), hip.DeviceArray.from_numpy(vals)
    hip.bitonic_merge_kv(dk, dv, m, batch)
    gk, gv = dk.numpy(), dv.numpy()
    for b in range(batch):
        ek, ev = O.bitonic_warp_merge(keys[b], vals[b], 32)
        assert np.array_equal(gk[b], ek) and np.array_equal(gv[b], ev), (m, b)


@pytest.mark.parametrize("bitlen", [8, 10, 13])
def test_hashmap_bit_exact(hip, bitlen):
    from oracle import oracle as O
    rng = np.random.default_rng(bitlen)
    size = 1 << bitlen
    keys = rng.integers(0, size * 3 // 4, size + 200).astype(np.uint32)  # repeats, long probe chains, then full
    keys[5] = 0x7FFFFFFF
    table = np.full(size, 0xFFFFFFFF, np.uint32)
    dt, dkeys = hip.DeviceArray.from_numpy(table), hip.DeviceArray.from_numpy(keys)
    dflags = hip.DeviceArray(keys.size, np.uint32)
    hip.hashmap_insert_seq(dt, bitlen, dkeys, keys.size, dflags)
    eflags, etable = O.hashmap_insert_seq(bitlen, keys)
    assert np.array_equal(dflags.numpy(), eflags)
    assert np.array_equal(dt.numpy(), etable)
    # fill the table completely: further new keys are refused, stored ones recognised
    fill = np.arange(size + 50, dtype=np.uint32) + 1000
    dfill = hip.DeviceArray.from_numpy(fill)
    dflags2 = hip.DeviceArray(fill.size, np.uint32)
    hip.hashmap_insert_seq(dt, bitlen, dfill, fill.size, dflags2)
    eflags2, etable2 = O.hashmap_insert_seq(bitlen, fill, etable.copy())
    assert np.array_equal(dflags2.numpy(), eflags2) and np.array_equal(dt.numpy(), etable2)
    assert (etable2 != 0xFFFFFFFF).all()


@pytest.mark.parametrize("dim", [4, 96, 128, 132, 960, 1024])
def test_distance_within_tolerance(hip, dim):
    from oracle import oracle as O
    rng = np.random.default_rng(dim)
    n = 257
    a = rng.standard_normal((n, dim)).astype(np.float32)
    b = rng.standard_normal((n, dim)).astype(np.float32)
    da, db, dout = hip.DeviceArray.from_numpy(a), hip.DeviceArray.from_numpy(b), hip.DeviceArray(n, np.float32)
    for metric in (O.EUCLIDEAN, O.COSINE):
        hip.distance_batch(da, db, n, dim, metric, dout)
        got = dout.numpy()
        ref = O.distance_batch(a, b, metric)
        assert np.allclose(got, ref, rtol=1e-5, atol=0), (dim, metric, np.abs(got / ref - 1).max())  # north-star tolerance
        exact = ((a.astype(np.float64) - b.astype(np.float64)) ** 2).sum(1)
        assert np.allclose(got, np.sqrt(exact) if metric == O.EUCLIDEAN else exact, rtol=1e-5)


def test_distance_integer_data_bit_exact(hip):
    from oracle import oracle as O
    rng = np.random.default_rng(1)
    n, dim = 512, 128
    a = rng.integers(0, 256, (n, dim)).astype(np.float32)
    b = rng.integers(0, 256, (n, dim)).astype(np.float32)
    b[:4] = a[:4]  # zero distances
    da, db, dout = hip.DeviceArray.from_numpy(a), hip.DeviceArray.from_numpy(b), hip.DeviceArray(n, np.float32)
    for metric in (O.EUCLIDEAN, O.COSINE):
        hip.distance_batch(da, db, n, dim, metric, dout)
        assert np.array_equal(dout.numpy(), O.distance_batch(a, b, metric))


def test_argument_errors(hip):
    d = hip.DeviceArray(16, np.float32)
    with pytest.raises(hip.GlideHipError) as e:
        hip.distance_batch(d, d, 1, 6, 0, d)       # dim not a multiple of 4
    assert e.value.code == -1
    with pytest.raises(hip.GlideHipError) as e:
        hip.bitonic_sort_kv(d, d, 96, 1)           # not a power-of-two network
    assert e.value.code == -1
    with pytest.raises(hip.GlideHipError) as e:
        hip.distance_batch(None, d, 1, 4, 0, d)
    assert e.value.code == -2


@pytest.mark.parametrize("count", [1, 3, 4, 127, 128, 1000003])
def test_widen_u8(hip, count):
    src = np.random.default_rng(count).integers(0, 256, size=count + 3, dtype=np.uint8)
    d_src = hip.DeviceArray.from_numpy(src)
    d_dst = hip.DeviceArray.full((count + 1,), -1.0, np.float32)
    hip.widen_u8(d_src, count, d_dst)
    hip.synchronize()
    out = d_dst.numpy()
    np.testing.assert_array_equal(out[:count], src[:count].astype(np.float32))
    assert out[count] == -1.0
