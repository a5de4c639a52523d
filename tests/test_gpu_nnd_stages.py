"""NN-descent one stage at a time: reverse sampling, local join and merge against a plain numpy/Python model.

Integer-valued rows (0..255, 128 dims) make every fp16 product and fp32 sum exact, so the join's distances, its
arg-min choices (smaller distance, then earlier position) and therefore its offers are bit-exact; the merge is a
deterministic function of its inputs and is compared field by field.
"""
from collections import Counter

import numpy as np
import pytest

from conftest import lowdim_data

pytestmark = pytest.mark.gpu
INV = 0xFFFFFFFF
OLD = 0x80000000
S = 32   # samples per list (NUM_SAMPLES, nn_descent.cuh:391)


@pytest.fixture(scope="module")
def hip():
    from glide_amd import capi
    capi.set_device(0)
    return capi


class Workspace:
    def __init__(self, hip, num, dim, degree):
        self.hip, self.num = hip, num
        self.l = hip.nnd_layout(num, dim, degree)
        self.bytes = hip.nnd_workspace_bytes(num, dim, degree)
        assert self.bytes == self.l.total
        self.buf = hip.DeviceArray(self.bytes // 4 + 1, np.uint32)

    def read(self):
        w, l, n = self.buf.numpy(), self.l, self.num
        def f(off, count, dtype=np.uint32):
            return w[off // 4: off // 4 + count].view(dtype).copy()
        return dict(
            list_ids=f(l.list_ids, n * l.width).reshape(n, l.width), list_dists=f(l.list_dists, n * l.width, np.float32).reshape(n, l.width),
            fwd_new=f(l.fwd_new, n * S).reshape(n, S), fwd_old=f(l.fwd_old, n * S).reshape(n, S),
            rev_new=f(l.rev_new, n * S).reshape(n, S), rev_old=f(l.rev_old, n * S).reshape(n, S),
            counts=f(l.counts, n * 4).reshape(n, 4), inbox_counts=f(l.inbox_counts, n),
            segment_state=f(l.segment_state, 16), segment_updates=f(l.segment_updates, 16),
            inbox=f(l.inbox, n * l.inbox_cap * 2).reshape(n, l.inbox_cap, 2), bloom=f(l.bloom, n * l.bloom_sets * 16).reshape(n, l.bloom_sets * 16),
            norms=f(l.norms, n, np.float32))


def _dedupe(first, second, limit):
    out, seen = [], set()
    for v in list(first) + list(second):
        v = int(v)
        if v < limit and v not in seen:
            seen.add(v)
            out.append(v)
    return out


def model_join(st, rows, seg_start, seg_len):
    """Offers of local_join_kernel (nn_descent.cuh:668-914): per list, each new member's nearest new and nearest old
    partner, each old member's nearest new partner.  Returns {target: sorted [(dist, cand)]} in reorder ids' partition-local space."""
    offers = {}
    half = rows.astype(np.float16).astype(np.float32)
    norms = (rows.astype(np.float32) ** 2).sum(1, dtype=np.float32)
    for node in range(seg_start, seg_start + seg_len):
        c = st["counts"][node]
        new = _dedupe(st["fwd_new"][node, :c[0]], st["rev_new"][node, :min(c[2], S)], seg_len)
        old = _dedupe(st["fwd_old"][node, :c[1]], st["rev_old"][node, :min(c[3], S)], seg_len)
        if not new:
            continue
        xn, nn_ = half[seg_start + np.array(new)], norms[seg_start + np.array(new)]
        d = np.maximum(nn_[:, None] + nn_[None, :] - 2.0 * (xn @ xn.T), 0.0).astype(np.float32)
        for i, a in enumerate(new):
            best, bj = None, None
            for j, b in enumerate(new):
                if j != i and (best is None or d[i, j] < best):
                    best, bj = d[i, j], b
            if bj is not None and bj != a:
                offers.setdefault(a, []).append((float(best), bj))
        if old:
            xo, no_ = half[seg_start + np.array(old)], norms[seg_start + np.array(old)]
            d = np.maximum(nn_[:, None] + no_[None, :] - 2.0 * (xn @ xo.T), 0.0).astype(np.float32)
            for i, a in enumerate(new):
                best, bj = None, None
                for j, b in enumerate(old):
                    if b != a and (best is None or d[i, j] < best):
                        best, bj = d[i, j], b
                if bj is not None:
                    offers.setdefault(a, []).append((float(best), bj))
            for j, b in enumerate(old):
                best, bi = None, None
                for i, a in enumerate(new):
                    if a != b and (best is None or d[i, j] < best):
                        best, bi = d[i, j], a
                if bi is not None:
                    offers.setdefault(b, []).append((float(best), bi))
    return {k: sorted(v) for k, v in offers.items()}


def _bloom_bits(key, sets):
    m = 0xFFFFFFFF
    def mix(v, a, c):
        v = (v * a + c) & m
        v ^= (v << 13) & m
        v ^= v >> 17
        v ^= (v << 5) & m
        return v
    base = (key % sets) * 512
    h = mix(key, 1103515245, 12345)        # BloomFilter hashes, nn_descent.cuh:203-276
    h1 = mix(key, 1664525, 1013904223)
    bits = [base + h % 512]
    h = (h + h1) & m
    bits.append(base + h % 512)
    h = (h + h1) & m
    bits.append(base + h % 512)
    return bits


def model_merge(st, node, width, cap, sets):
    """One node of the merge stage; returns (list_ids, list_dists, fwd_new, n_new, fwd_old, n_old, bloom words,
    number of offers that entered the list)."""
    ids, dists = [int(v) for v in st["list_ids"][node]], st["list_dists"][node]
    fwd_old = [v & ~OLD for v in ids if v != INV and v & OLD]
    n_in = min(int(st["inbox_counts"][node]), cap)
    ent = []   # (dist bits, id, source, flag)
    for v, d in zip(ids, dists):
        if v != INV:
            ent.append((int(np.float32(d).view(np.uint32)), v & ~OLD, 0, v & OLD))
    for db, cand in st["inbox"][node, :n_in]:
        ent.append((int(db), int(cand), 1, 0))
    ent.sort(key=lambda e: (e[0], e[1], e[2]))
    words = st["bloom"][node].copy()
    seen_before = words.copy()
    out, fwd_new, rank = [], [], 0
    prev = None
    for e in ent:
        same = prev is not None and prev[0] == e[0] and prev[1] == e[1]
        if e[2] == 0:
            if not same:
                out.append((e[1] | e[3], e[0], 0))
        elif not same or prev[2] == 0:          # first offered copy of this id
            known = same
            if rank < S:
                bits = _bloom_bits(e[1], sets)
                fresh = not all((int(seen_before[b >> 5]) >> (b & 31)) & 1 for b in bits)
                if fresh:
                    fwd_new.append(e[1])
                    for b in bits:
                        words[b >> 5] |= np.uint32(1 << (b & 31))
                if not known:
                    out.append((e[1] | (OLD if fresh else 0), e[0], 1))
            rank += 1
        prev = e
    out = out[:width]
    l_ids = np.full(width, INV, np.uint32)
    l_d = np.full(width, np.finfo(np.float32).max, np.float32)
    inserted = sum(o[2] for o in out)
    for i, (v, db, _) in enumerate(out):
        l_ids[i] = v
        l_d[i] = np.array([db], np.uint32).view(np.float32)[0]
    return l_ids, l_d, fwd_new, len(fwd_new), fwd_old[:S], min(len(fwd_old), S), words, inserted


@pytest.mark.parametrize("degree", [32, 64])
def test_stages_match_model(hip, degree):
    num, dim = 2400, 128
    rows = lowdim_data(num, dim, seed=5)
    seg_start, seg_len = np.array([0, 1500], np.uint32), np.array([1500, 900], np.uint32)
    d_rows = hip.DeviceArray.from_numpy(rows)
    d_ss, d_sl = hip.DeviceArray.from_numpy(seg_start), hip.DeviceArray.from_numpy(seg_len)
    ws = Workspace(hip, num, dim, degree)
    args = (num, dim, d_ss, d_sl, 2, degree, ws.buf, ws.bytes)
    hip.nnd_prepare(d_rows, num, dim, d_ss, d_sl, 2, degree, 3, ws.buf, ws.bytes)
    hip.synchronize()
    st = ws.read()
    width, cap, sets = ws.l.width, ws.l.inbox_cap, ws.l.bloom_sets
    # prepare: random partition-local ids, no self, all sampled (flagged) as the first "new" samples
    local = np.arange(num) - np.repeat(seg_start, seg_len)
    lim = np.repeat(seg_len, seg_len)[:, None]
    assert ((st["list_ids"] & ~np.uint32(OLD)) < lim).all()
    assert ((st["list_ids"] & ~np.uint32(OLD)) != local[:, None]).all()
    assert (st["counts"][:, 0] == S).all() and (st["counts"][:, 1] == 0).all()
    np.testing.assert_array_equal(st["norms"], (rows ** 2).sum(1, dtype=np.float32))

    for it in range(3):
        print("degree", degree, "round", it, flush=True)
        hip.nnd_reverse_sample(*args)
        hip.synchronize()
        st = ws.read()
        # reverse samples: v in fwd(u)  <=>  u arrives at rev(v); arrivals counted, the first 32 stored (any order)
        for which, fwd, rev in ((0, "fwd_new", "rev_new"), (1, "fwd_old", "rev_old")):
            expect = {}
            for s0, l0 in zip(seg_start, seg_len):
                for u in range(s0, s0 + l0):
                    for v in st[fwd][u, :st["counts"][u, which]]:
                        expect.setdefault(int(s0 + v), []).append(int(u - s0))
            for v in range(num):
                e = expect.get(v, [])
                assert st["counts"][v, 2 + which] == len(e)
                got = Counter(st[rev][v, :min(len(e), S)].tolist())
                assert not got - Counter(e)          # a sub-multiset of the arrivals
                if len(e) <= S:
                    assert got == Counter(e)
        assert (st["inbox_counts"] == 0).all()

        hip.nnd_local_join(*args)
        hip.synchronize()
        after = ws.read()
        total = 0
        for s0, l0 in zip(seg_start.tolist(), seg_len.tolist()):
            offers = model_join(st, rows, s0, l0)
            for t in range(l0):
                exp = offers.get(t, [])
                cnt = int(after["inbox_counts"][s0 + t])
                assert cnt == len(exp), (s0, t, cnt, len(exp))
                got = sorted((float(np.array([db], np.uint32).view(np.float32)[0]), int(c)) for db, c in after["inbox"][s0 + t, :min(cnt, cap)])
                if cnt <= cap:
                    assert got == exp, (s0, t)
                else:
                    assert all(g in exp for g in got)
                total += cnt
        assert total > 0

        hip.nnd_merge(*args)
        hip.synchronize()
        merged = ws.read()
        updates = [0, 0]
        for node in range(num):
            l_ids, l_d, fn, n_new, fo, n_old, words, inserted = model_merge(after, node, width, cap, sets)
            if node % 100 == 0:
                updates[0 if node < seg_len[0] else 1] += inserted
            np.testing.assert_array_equal(merged["list_ids"][node], l_ids, err_msg="list ids of node %d" % node)
            np.testing.assert_array_equal(merged["list_dists"][node], l_d)
            assert merged["counts"][node].tolist() == [n_new, n_old, 0, 0]
            assert merged["fwd_new"][node, :n_new].tolist() == fn
            assert merged["fwd_old"][node, :n_old].tolist() == fo
            np.testing.assert_array_equal(merged["bloom"][node], words)
        assert (merged["inbox_counts"] == 0).all()
        assert merged["segment_updates"][:2].tolist() == updates
        # termination test: limit = threshold * rows * dim / 100; a partition below it gets one more round, then rests
        threshold = [0.0, 1e9, 1e9][it]
        before = merged["segment_state"][:2].tolist()
        hip.nnd_converge(num, dim, d_ss, d_sl, 2, degree, threshold, ws.buf, ws.bytes)
        hip.synchronize()
        st = ws.read()
        expect = [2 if b == 1 else (1 if b == 0 and u < threshold * num * dim / 100 else b) for b, u in zip(before, updates)]
        assert st["segment_state"][:2].tolist() == expect and st["segment_updates"][:2].tolist() == [0, 0]
        assert expect == [[0, 0], [1, 1], [2, 2]][it]

    # a resting partition is skipped by every stage
    hip.nnd_reverse_sample(*args)
    hip.nnd_local_join(*args)
    hip.nnd_merge(*args)
    hip.synchronize()
    rest = ws.read()
    for key in ("list_ids", "list_dists", "fwd_new", "fwd_old", "bloom", "inbox_counts"):
        np.testing.assert_array_equal(rest[key], st[key], err_msg=key)

    d_knn = hip.DeviceArray((num, degree), np.uint32)
    hip.nnd_finalize(num, dim, d_ss, d_sl, 2, degree, d_knn, None, ws.buf, ws.bytes)
    hip.synchronize()
    knn = d_knn.numpy()
    valid = st["list_ids"][:, :degree] != INV
    np.testing.assert_array_equal(knn[valid], (st["list_ids"][:, :degree] & ~np.uint32(OLD))[valid])
    assert (knn < lim).all()
