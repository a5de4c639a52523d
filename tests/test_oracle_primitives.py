"""Pins of the CPU oracle's primitives against facts that do not come from the oracle itself."""
import itertools

import numpy as np
import pytest

from oracle import oracle as O


# ---------------------------------------------------------------- params (reference params.cuh:49-99)
def test_search_param_table():
    # hand-computed: max_iter = 1 + min(1.1*beam, beam+10) truncated; hash bits = smallest b >= 8 with
    # beam + degree <= 2^b / 2; reset = largest r with beam + degree*(r+1) <= 2^b / 2 ... +1 step past
    expect = {  # (beam, degree): (max_iter, hash_bit, reset)
        (32, 32): (36, 8, 3), (64, 32): (71, 8, 2), (128, 32): (139, 9, 4), (256, 32): (267, 10, 8),
        (64, 64): (71, 8, 1), (128, 64): (139, 9, 2), (256, 64): (267, 10, 4),
    }
    for (beam, degree), (mi, hb, rs) in expect.items():
        sp = O.search_params(beam, degree)
        assert (sp["max_iterations"], sp["hash_bit"], sp["hash_reset_interval"]) == (mi, hb, rs), (beam, degree, sp)


def test_beam_rounding_and_closed_forms():
    for beam in range(1, 300, 7):
        mi, b = O.adjust_search_params(0, 0, beam)
        assert b == ((beam + 31) // 32) * 32
        assert mi == 1 + int(min(beam * 1.1, beam + 10.0))
    # user-given max_iterations is kept when larger, min_iterations lifts it
    assert O.adjust_search_params(0, 500, 64)[0] == 500
    assert O.adjust_search_params(90, 0, 64)[0] == 90  # 0 < min_iterations lifts the derived value to min_iterations
    for beam, deg in itertools.product((32, 64, 100, 500, 3000), (32, 64, 200)):
        hb = O.hash_bitlen(beam, deg)
        assert 8 <= hb <= 13
        if hb < 13:
            assert beam + deg <= (1 << hb) * 0.5 and (hb == 8 or beam + deg > (1 << (hb - 1)) * 0.5)


def test_nnd_degree_and_xorshift():
    assert [O.nnd_extended_degree(k) for k in (16, 32, 33, 48, 64)] == [32, 32, 64, 64, 96]

    def ref(u):  # utils.cuh:14-19 in plain python ints
        u &= 0xFFFFFFFF
        u ^= u >> 13
        u ^= (u << 27) & 0xFFFFFFFF
        u ^= u >> 5
        return (u * 0x9E3779B9) & 0xFFFFFFFF
    for x in (0, 1, 12345, 0xFFFFFFFF, 0x80000000):
        assert O.xorshift32(x) == ref(x)


# ---------------------------------------------------------------- bitonic network
@pytest.mark.parametrize("m", [32, 64, 128, 256, 512])
def test_bitonic_sorts_distinct_keys(m):
    rng = np.random.default_rng(m)
    for _ in range(20):
        keys = rng.permutation(m).astype(np.float32)
        vals = (keys * 3 + 1).astype(np.uint32)
        k, v = O.bitonic_warp_sort(keys, vals)
        assert np.array_equal(k, np.sort(keys))
        assert np.array_equal(v, (k * 3 + 1).astype(np.uint32))


def test_bitonic_zero_one_principle_small():
    # a comparator network sorts every input iff it sorts every 0/1 input; exhaustive on M = 32 is 2^32, so
    # check all 0/1 inputs with at most 3 ones or at most 3 zeros plus 20000 random ones (values track keys)
    m = 32
    rng = np.random.default_rng(0)
    cases = []
    for ones in range(4):
        for pos in itertools.combinations(range(m), ones):
            a = np.zeros(m, np.float32)
            a[list(pos)] = 1
            cases.append(a)
            cases.append(1 - a)
    cases += [rng.integers(0, 2, m).astype(np.float32) for _ in range(20000)]
    for a in cases:
        k, _ = O.bitonic_warp_sort(a, np.arange(m, dtype=np.uint32))
        assert np.all(np.diff(k) >= 0)


def test_bitonic_ties_keep_a_permutation():
    rng = np.random.default_rng(5)
    for m in (64, 128):
        keys = rng.integers(0, 6, m).astype(np.float32)
        vals = np.arange(m, dtype=np.uint32)
        k, v = O.bitonic_warp_sort(keys, vals)
        assert np.all(np.diff(k) >= 0)
        assert sorted(v.tolist()) == list(range(m))
        assert np.array_equal(keys[v], k)  # each value still travels with its own key


def test_bitonic_equal_keys_never_move():
    # all keys equal: the compare-exchange is a no-op (bitonic.cuh:26), so values stay where they were
    vals = np.random.default_rng(1).permutation(128).astype(np.uint32)
    k, v = O.bitonic_warp_sort(np.full(128, 7.0, np.float32), vals)
    assert np.array_equal(v, vals)


def test_bitonic_merge_of_bitonic_input():
    rng = np.random.default_rng(9)
    for m in (64, 256):
        up = np.sort(rng.permutation(1000)[:m // 2]).astype(np.float32)
        down = np.sort(rng.permutation(1000)[:m // 2] + 1000)[::-1].astype(np.float32)
        keys = np.concatenate([up, down])
        k, _ = O.bitonic_warp_merge(keys, np.arange(m, dtype=np.uint32), 32)
        assert np.array_equal(k, np.sort(keys))


def test_sort_with_key_value_strided_layout():
    # distinct keys -> plain ascending order whatever the load permutation; fewer items than the network size
    rng = np.random.default_rng(3)
    for mx, n in ((32, 16), (32, 32), (64, 40), (256, 200)):
        keys = rng.permutation(n).astype(np.float32) + 0.5
        v, k = O.sort_with_key_value(mx, np.arange(n, dtype=np.uint32), keys)
        assert np.array_equal(k, np.sort(keys))
        assert np.array_equal(keys[v], k)


# ---------------------------------------------------------------- hashmap (reference hashmap.cuh:23-56)
def test_hashmap_hand_derived_layout():
    # bitlen 8: slot = (key ^ key >> 8) & 255, linear probing
    flags, table = O.hashmap_insert_seq(8, [5, 261, 5, 0x105 ^ 0x100, 517])
    # 5 -> slot 5; 261 = 0x105 -> (0x105 ^ 1) & 255 = 4; 5 again -> present; 0x005 -> same key 5 -> present;
    # 517 = 0x205 -> (0x205 ^ 2) & 255 = 7
    assert flags.tolist() == [1, 1, 0, 0, 1]
    assert table[5] == 5 and table[4] == 261 and table[7] == 517
    assert (table != 0xFFFFFFFF).sum() == 3
    # collision chain: 0 -> slot 0, 256 -> (0x100 ^ 1) = slot 1, 257 -> (0x101 ^ 1) & 255 = slot 0 -> probes to 2
    flags, table = O.hashmap_insert_seq(8, [0, 256, 257])
    assert flags.tolist() == [1, 1, 1] and table[0] == 0 and table[1] == 256 and table[2] == 257


def test_hashmap_set_invariants_and_full_table():
    rng = np.random.default_rng(2)
    keys = rng.integers(0, 200, 600).astype(np.uint32)
    flags, table = O.hashmap_insert_seq(9, keys)
    seen = set()
    for k, f in zip(keys.tolist(), flags.tolist()):
        assert f == (0 if k in seen else 1)
        seen.add(k)
    assert set(table[table != 0xFFFFFFFF].tolist()) == seen
    # a full table rejects new keys and still recognises stored ones
    keys = np.arange(300, dtype=np.uint32)
    flags, table = O.hashmap_insert_seq(8, keys)
    assert flags[:256].all() and not flags[256:].any()
    again, _ = O.hashmap_insert_seq(8, keys[:10], table.copy())
    assert not again.any()


# ---------------------------------------------------------------- distance (reference distance.cuh:9-27)
@pytest.mark.parametrize("dim", [4, 31, 96, 128, 960, 1000])
def test_distance_closed_form(dim):
    rng = np.random.default_rng(dim)
    a = rng.standard_normal((50, dim)).astype(np.float32)
    b = rng.standard_normal((50, dim)).astype(np.float32)
    sq = ((a.astype(np.float64) - b.astype(np.float64)) ** 2).sum(1)
    got_l2 = O.distance_batch(a, b, O.EUCLIDEAN)
    got_cos = O.distance_batch(a, b, O.COSINE)
    assert np.allclose(got_l2, np.sqrt(sq), rtol=1e-5)
    assert np.allclose(got_cos, sq, rtol=1e-5)


def test_distance_cosine_identity_and_integer_exactness():
    rng = np.random.default_rng(0)
    a = rng.standard_normal((20, 96))
    b = rng.standard_normal((20, 96))
    a /= np.linalg.norm(a, axis=1, keepdims=True)
    b /= np.linalg.norm(b, axis=1, keepdims=True)
    got = O.distance_batch(a.astype(np.float32), b.astype(np.float32), O.COSINE)
    assert np.allclose(got, 2 - 2 * (a * b).sum(1), atol=2e-6)  # squared L2 of unit rows = 2 - 2 cos
    x = rng.integers(0, 256, (20, 128)).astype(np.float32)
    y = rng.integers(0, 256, (20, 128)).astype(np.float32)
    exact = ((x.astype(np.int64) - y.astype(np.int64)) ** 2).sum(1)
    assert np.array_equal(O.distance_batch(x, y, O.COSINE), exact.astype(np.float32))  # sums stay below 2^24
    assert np.array_equal(O.distance_batch(x, y, O.EUCLIDEAN), np.sqrt(exact.astype(np.float64)).astype(np.float32))


def _swz(j):
    return j ^ (j >> 5)


@pytest.mark.parametrize("max_cand,degree,beam", [(64, 32, 32), (64, 64, 200), (128, 96, 64), (128, 128, 300), (256, 160, 64),
                                                  (256, 256, 100), (256, 200, 256), (256, 256, 512), (256, 130, 130)])
def test_sort_for_candidate_selects_the_smallest(max_cand, degree, beam):
    """Distinct keys: the first min(degree, beam) slots (swizzled) end up holding the smallest candidates in ascending
    order, for the one-warp (search_kernel.cuh:9-37) and the two-warp (:38-94) variant alike."""
    rng = np.random.default_rng(max_cand + degree + beam)
    size = 1024
    dist = np.full(size, np.float32(3e38))
    ids = np.full(size, 0xFFFFFFFF, np.uint32)
    dist[:degree] = rng.permutation(degree * 4)[:degree].astype(np.float32)
    ids[:degree] = np.arange(degree) + 1000
    d, i = O.sort_for_candidate(max_cand, dist, ids, degree, beam)
    keep = min(degree, beam)
    order = np.argsort(dist[:degree])[:keep]
    got_d = np.array([d[_swz(j)] for j in range(keep)])
    got_i = np.array([i[_swz(j)] for j in range(keep)])
    np.testing.assert_array_equal(got_d, dist[:degree][order])
    np.testing.assert_array_equal(got_i, ids[:degree][order])


@pytest.mark.parametrize("max_beam,beam,degree", [(64, 64, 32), (128, 100, 64), (256, 256, 128), (256, 200, 32), (512, 512, 32),
                                                  (512, 300, 64), (512, 400, 256), (512, 512, 256), (512, 258, 32)])
def test_sort_for_beam_merges_to_the_smallest(max_beam, beam, degree):
    """Distinct keys, even beam: the beam after the merge is the ascending list of the `beam` smallest of beam + candidates,
    for the one-warp (search_kernel.cuh:97-148) and the two-warp (:149-232) variant alike; repeated over several rounds
    so that the two-warp variant's turning points start from every kind of previous state."""
    rng = np.random.default_rng(max_beam + beam + degree)
    max_cand = 64 if degree <= 64 else 128 if degree <= 128 else 256
    size = 2048
    pool = rng.permutation(100000).astype(np.float32)
    used = 0
    bd = np.full(size, np.float32(3e38))
    bi = np.full(size, 0xFFFFFFFF, np.uint32)
    truth = []
    for rnd in range(6):
        n_valid = int(rng.integers(0, degree + 1))
        cd = np.full(size, np.float32(3e38))
        ci = np.full(size, 0xFFFFFFFF, np.uint32)
        cd[:n_valid] = pool[used:used + n_valid] * (0.2 if rnd % 2 else 1.0)
        ci[:n_valid] = np.arange(used, used + n_valid)
        used += n_valid
        cd[:n_valid] += np.arange(n_valid) * 1e-3 * 0          # keys stay distinct integers or fifths
        # make keys distinct against everything seen so far
        seen = {k for k, _ in truth}
        for t in range(n_valid):
            while float(cd[t]) in seen:
                cd[t] += 0.5
            seen.add(float(cd[t]))
        cand = sorted(zip(cd[:n_valid].tolist(), ci[:n_valid].tolist()))
        sd, si = O.sort_for_candidate(max_cand, cd, ci, degree, beam)
        bd, bi = O.sort_for_beam(max_beam, bd, bi, beam, sd, si, degree, rnd == 0)
        truth = sorted(truth + cand)[:beam] if rnd else cand[:beam]
        got = [(float(bd[_swz(j)]), int(bi[_swz(j)])) for j in range(len(truth))]
        assert got == [(float(np.float32(k)), v) for k, v in truth], (rnd, max_beam, beam, degree)
        for j in range(len(truth), beam):
            assert bd[_swz(j)] >= np.float32(3e38)


def test_sort_of_32_slots_on_the_64_network_equals_the_32_network():
    """With at most 32 candidate slots in use, the reference's strided load (search_kernel.cuh:9-37) puts them on the
    even elements of the 64-element network and +inf on the odd ones.  The sorted sequence, ties included, is the one
    the 32-element network gives on the slots alone, provided every +inf key carries the invalid id; the GPU code
    relies on this.  A real id with an +inf key is the exception (shown too)."""
    from oracle import oracle as O
    rng = np.random.default_rng(3)
    fmax = np.finfo(np.float32).max
    exception_seen = False
    for trial in range(3000):
        used = int(rng.integers(1, 33))
        keys = np.full(32, fmax, np.float32)
        vals = np.full(32, 0xFFFFFFFF, np.uint32)
        keys[:used] = rng.integers(0, rng.integers(1, 7), used).astype(np.float32)      # many equal keys
        vals[:used] = rng.permutation(100000)[:used].astype(np.uint32)
        dead = rng.random(32) < rng.random() * 0.5                                       # visited / empty graph slots
        keys[dead], vals[dead] = fmax, 0xFFFFFFFF
        k64, v64 = np.full(64, fmax, np.float32), np.full(64, 0xFFFFFFFF, np.uint32)
        k64[0::2], v64[0::2] = keys, vals
        a_k, a_v = O.bitonic_warp_sort(k64, v64)
        b_k, b_v = O.bitonic_warp_sort(keys, vals)
        assert np.array_equal(a_k[:32], b_k) and np.array_equal(a_v[:32], b_v), trial
        assert (a_k[32:] == fmax).all() and (a_v[32:] == 0xFFFFFFFF).all()
        # a real id under an +inf key may end up anywhere among the +inf keys of the larger network
        keys2, vals2 = keys.copy(), vals.copy()
        j = int(rng.integers(0, 32))
        keys2[j], vals2[j] = fmax, 77
        k64[0::2], v64[0::2] = keys2, vals2
        a_k, a_v = O.bitonic_warp_sort(k64, v64)
        b_k, b_v = O.bitonic_warp_sort(keys2, vals2)
        exception_seen |= not np.array_equal(a_v[:32], b_v)
    assert exception_seen
