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
R = 256  # words of a reverse overflow table: 16 buckets of 15 slots + the bucket's bound
SLOTS = 256  # slots of a node's offer table when the list is one sub-list; 512 with several.  Every offer goes to two slots of one line
RCAP = 64  # reverse samples a list holds before the overflow table takes over


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
            rev_new=f(l.rev_new, n * l.reverse_stride).reshape(n, l.reverse_stride)[:, :RCAP], rev_old=f(l.rev_old, n * l.reverse_stride).reshape(n, l.reverse_stride)[:, :RCAP],
            rev_tables=f(l.rev_tables, n * 2 * R).reshape(n, 2, R), counts=f(l.counts, n * 4).reshape(n, 4),
            rev_thr=f(l.rev_thr, n * 2).reshape(n, 2),
            segment_state=f(l.segment_state, 16), segment_updates=f(l.segment_updates, 16), round=int(f(l.round, 1)[0]),
            offers=f(l.offers, n * l.offer_slots * 2).view(np.uint64).reshape(n, l.offer_slots),
            bloom=f(l.bloom, n * l.bloom_sets * 16).reshape(n, l.bloom_sets * 16),
            norms=f(l.norms, 2 * n, np.float32)[0::2].copy(), offer_thr=f(l.norms, 2 * n)[1::2].copy())


NO_OFFER = np.uint64(0xFFFFFFFFFFFFFFFF)
SLOT = np.arange(256) % 16 != 15          # word 15 of every bucket of 16 is the bucket's bound, the others are slots


def offer_key(dist, cand):
    return (int(np.float32(dist).view(np.uint32)) << 32) | int(cand)


def table_slots(row):
    """(slot values that are not empty, sorted; the bucket bounds) of one table row as read from the device."""
    row = np.asarray(row)
    empty = NO_OFFER if row.dtype == np.uint64 else np.uint32(INV)
    slots = row[SLOT[:row.size]]
    return sorted(int(x) for x in slots[slots != empty]), [int(x) for x in row[15::16]]


def reverse_samples(st, node, which):
    """The 32 smallest sources that arrived at `node`: its list (the first 64 arrivals) and, beyond 64 arrivals, its overflow table.
    A source whose list holds `node` twice (the start lists of a partition hardly larger than a list do: init_random_graph
    replaces a node's own id by the entry 32 places on, nn_descent.cuh:1003-1038) arrives twice and counts twice, as in a
    sweep over the lists in order (add_rev_edges_kernel :490-507)."""
    cnt = int(st["counts"][node, 2 + which])
    got = [int(x) for x in st[("rev_new", "rev_old")[which]][node, :min(cnt, RCAP)]]
    if cnt > RCAP:
        got += table_slots(st["rev_tables"][node, which])[0]
    return sorted(got)[:S]


def offers_held(st, node, distinct=True):
    """The offers a node's table holds after a join, ascending."""
    row = st["offers"][node]
    held = [int(x) for x in row[row != NO_OFFER]]
    return sorted(set(held) if distinct else held)


def model_offer_table(keys, round_, slots=SLOTS):
    """What a node's offer table holds once `keys` (distance bits << 32 | candidate) have all been sent to it: a slot
    keeps the smallest key it was sent.  With x = candidate ^ round * 0x85EBCA6B a key goes to slot
    s1 = (x * 0x9E3779B1) >> (32 - log2 slots) and to a second slot of the same line of 16,
    (s1 & ~15) | ((s1 + 1 + ((x * 0xC2B2AE35 mod 2^32) * 15 >> 32)) & 15)."""
    row = np.full(slots, NO_OFFER, np.uint64)
    salt = (round_ * 0x85EBCA6B) & 0xFFFFFFFF
    for key in keys:
        x, shift = (key & 0xFFFFFFFF) ^ salt, 32 - slots.bit_length() + 1
        s1 = ((x * 0x9E3779B1) & 0xFFFFFFFF) >> shift
        s2 = (s1 & ~15) | ((s1 + 1 + ((((x * 0xC2B2AE35) & 0xFFFFFFFF) * 15) >> 32)) & 15)
        for slot in (s1, s2):
            if key < int(row[slot]):
                row[slot] = np.uint64(key)
    return row


def model_offer_threshold(st, node):
    """The threshold a node announces for the next join: when five eighths of its table's slots or more were taken, the
    distance (bits) of the 64th best offer; one in force is kept while 40 or more slots are taken and 32 or more
    offers held."""
    taken, held = len(offers_held(st, node, distinct=False)), offers_held(st, node)
    if taken >= st["offers"].shape[1] * 5 // 8:
        return held[63] >> 32 if len(held) >= 64 else INV
    if taken >= 40 and len(held) >= S:
        return int(st["offer_thr"][node])
    return INV


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
        # forward samples in list order, then the 32 smallest reverse samples in ascending order
        new = _dedupe(st["fwd_new"][node, :c[0]], reverse_samples(st, node, 0), seg_len)
        old = _dedupe(st["fwd_old"][node, :c[1]], reverse_samples(st, node, 1), seg_len)
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
    # a node that overflowed has announced a threshold: offers that are not below it stay away
    return {k: sorted(o for o in v if offer_key(*o) >> 32 < int(st["offer_thr"][seg_start + k])) for k, v in offers.items()}


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


def model_merge(st, node, width, sets):
    """One node of the merge stage; returns (list_ids, list_dists, fwd_new, fwd_old, bloom words, number of offers that
    entered the list).  The list is width / 32 sub-lists keyed by id % (width / 32); entry r of sub-list s is slot
    r * (width / 32) + s (update_graph nn_descent.cuh:1106-1126, insert_to_ordered_list :916-943)."""
    num_sub = width // S
    ids, dists = [int(v) for v in st["list_ids"][node]], st["list_dists"][node]
    fwd_old = [v & ~OLD for v in ids if v != INV and v & OLD][:S]
    best = offers_held(st, node)[:S]      # the round's 32-wide device list
    held = {v & ~OLD for v in ids if v != INV}
    words, seen_before = st["bloom"][node].copy(), st["bloom"][node].copy()
    ent = [(int(np.float32(d).view(np.uint32)), v & ~OLD, 0, v & OLD) for v, d in zip(ids, dists) if v != INV]
    fwd_new = []
    for key in best:
        db, cand = key >> 32, key & 0xFFFFFFFF
        bits = _bloom_bits(cand, sets)
        fresh = not all((int(seen_before[b >> 5]) >> (b & 31)) & 1 for b in bits)
        if fresh:
            fwd_new.append(cand)
            for b in bits:
                words[b >> 5] |= np.uint32(1 << (b & 31))
        if cand not in held:          # an id the list holds is rejected whatever its distance there
            held.add(cand)
            ent.append((db, cand, 1, OLD if fresh else 0))
    ent.sort(key=lambda e: (e[0], e[1], e[2]))
    l_ids = np.full(width, INV, np.uint32)
    l_d = np.full(width, np.finfo(np.float32).max, np.float32)
    rank, inserted, prev = [0] * num_sub, 0, None
    for e in ent:
        if prev is not None and prev[:2] == e[:2]:
            continue                   # a repeated entry of a random start list
        prev = e
        s_ = e[1] % num_sub
        if rank[s_] < S:
            slot = rank[s_] * num_sub + s_
            l_ids[slot] = e[1] | e[3]
            l_d[slot] = np.array([e[0]], np.uint32).view(np.float32)[0]
            inserted += e[2]
        rank[s_] += 1
    return l_ids, l_d, fwd_new, fwd_old, words, inserted


@pytest.mark.parametrize("degree", [32, 64, 96, 128])
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
    width, sets = ws.l.width, ws.l.bloom_sets
    num_sub = width // S
    assert width == {32: 32, 64: 96, 96: 128, 128: 192}[degree] and ws.l.offer_slots == (256 if degree == 32 else 512)
    # prepare: random partition-local ids, no self, sub-list s holds ids = s mod num_sub; the first 32 in storage
    # order are sampled (flagged) as the first "new" samples
    local = np.arange(num) - np.repeat(seg_start, seg_len)
    lim = np.repeat(seg_len, seg_len)[:, None]
    assert ((st["list_ids"] & ~np.uint32(OLD)) < lim).all()
    assert ((st["list_ids"] & ~np.uint32(OLD)) != local[:, None]).all()
    assert (((st["list_ids"] & ~np.uint32(OLD)) % num_sub) == (np.arange(width) % num_sub)[None, :]).all()
    assert (st["counts"][:, 0] == S).all() and (st["counts"][:, 1] == 0).all()
    np.testing.assert_array_equal(st["fwd_new"], st["list_ids"][:, :S] & ~np.uint32(OLD))
    assert (st["offers"] == NO_OFFER).all() and (st["rev_tables"] == INV).all() and st["round"] == 0
    assert (st["counts"][:, 2:] == 0).all() and (st["rev_thr"] == INV).all() and (st["offer_thr"] == INV).all()
    np.testing.assert_array_equal(st["norms"], (rows ** 2).sum(1, dtype=np.float32))

    for it in range(3):
        print("degree", degree, "round", it, flush=True)
        hip.nnd_reverse_sample(*args)
        hip.synchronize()
        st = ws.read()
        # reverse samples: v in fwd(u)  <=>  u arrives at rev(v).  Every arrival is counted, the first 64 sit in the list,
        # later ones in the overflow table; what the join uses are the 32 smallest sources (what a sweep over the lists in
        # order keeps, add_rev_edges_kernel :490-507), whatever the order of arrival was
        overflowed = 0
        for which, fwd, rev in ((0, "fwd_new", "rev_new"), (1, "fwd_old", "rev_old")):
            expect = {}
            for s0, l0 in zip(seg_start, seg_len):
                for u in range(s0, s0 + l0):
                    for v in st[fwd][u, :st["counts"][u, which]]:
                        if u - s0 < st["rev_thr"][s0 + v, which]:       # sources not below a node's threshold stay away
                            expect.setdefault(int(s0 + v), []).append(int(u - s0))
            for v in range(num):
                e = sorted(expect.get(v, ()))
                assert st["counts"][v, 2 + which] == len(e)
                assert not Counter(st[rev][v, :min(len(e), RCAP)].tolist()) - Counter(e)       # the list: a sub-multiset of the arrivals
                in_table, bounds = table_slots(st["rev_tables"][v, which])
                if len(e) <= RCAP:
                    assert not in_table and all(b == INV for b in bounds)
                else:
                    overflowed += 1
                    assert not Counter(in_table) - Counter(e)
                assert reverse_samples(st, v, which) == sorted(e)[:S]
        assert overflowed > 0 or it == 0 or degree > 32
        assert (st["offers"] == NO_OFFER).all() and st["round"] == it

        hip.nnd_local_join(*args)
        hip.synchronize()
        after = ws.read()
        assert (after["rev_tables"] == INV).all() and (after["counts"][:, 2:] == 0).all()      # consumed by the join
        # thresholds for the next scatter: after an overflow the 56th smallest source, kept while 40 or more still arrive
        for which in (0, 1):
            for v in range(num):
                cnt = int(st["counts"][v, 2 + which])
                if cnt > RCAP:
                    union = sorted(set([int(x) for x in st[("rev_new", "rev_old")[which]][v]] + table_slots(st["rev_tables"][v, which])[0]))
                    want = union[55] if len(union) >= 56 else INV
                else:
                    want = int(st["rev_thr"][v, which]) if cnt >= 40 else INV
                assert after["rev_thr"][v, which] == want, (which, v, cnt)
        total = sent = 0
        for s0, l0 in zip(seg_start.tolist(), seg_len.tolist()):
            offers = model_join(st, rows, s0, l0)
            for t in range(l0):
                # the table: per slot the smallest key sent there, whatever the order of arrival
                exp = model_offer_table([offer_key(d, c) for d, c in offers.get(t, [])], it, ws.l.offer_slots)
                np.testing.assert_array_equal(after["offers"][s0 + t], exp, err_msg="offer table of node %d" % (s0 + t))
                total += len(set(exp[exp != NO_OFFER].tolist()))
                sent += len(set(offers.get(t, [])))
        assert total > 0.8 * sent > 0          # few offers share a slot with a nearer one

        hip.nnd_merge(*args)
        hip.synchronize()
        merged = ws.read()
        updates = [0, 0]
        for node in range(num):
            l_ids, l_d, fn, fo, words, inserted = model_merge(after, node, width, sets)
            if node % 100 == 0:
                updates[0 if node < seg_len[0] else 1] += inserted
            np.testing.assert_array_equal(merged["list_ids"][node], l_ids, err_msg="list ids of node %d" % node)
            np.testing.assert_array_equal(merged["list_dists"][node], l_d)
            assert merged["counts"][node].tolist() == [len(fn), len(fo), 0, 0]
            assert merged["fwd_new"][node, :len(fn)].tolist() == fn
            assert merged["fwd_old"][node, :len(fo)].tolist() == fo
            np.testing.assert_array_equal(merged["bloom"][node], words)
        assert (merged["offers"] == NO_OFFER).all()
        assert merged["segment_updates"][:2].tolist() == updates
        for node in range(num):
            assert int(merged["offer_thr"][node]) == model_offer_threshold(after, node), node
        # lists: no id twice, never the node itself, every sub-list nearest first
        clean = merged["list_ids"] & ~np.uint32(OLD)
        for node in range(0, num, 7):
            row = clean[node][merged["list_ids"][node] != INV]
            assert len(set(row.tolist())) == row.size and (row != local[node]).all()
        for s_ in range(num_sub):
            assert (np.diff(merged["list_dists"][:, s_::num_sub], axis=1) >= 0).all()
        # termination test: limit = threshold * rows * dim / 100; a partition below it gets one more round, then rests
        threshold = [0.0, 1e9, 1e9][it]
        before = merged["segment_state"][:2].tolist()
        hip.nnd_converge(num, dim, d_ss, d_sl, 2, degree, threshold, ws.buf, ws.bytes)
        hip.synchronize()
        st = ws.read()
        expect = [2 if b == 1 else (1 if b == 0 and u < threshold * num * dim / 100 else b) for b, u in zip(before, updates)]
        assert st["segment_state"][:2].tolist() == expect and st["segment_updates"][:2].tolist() == [0, 0]
        assert expect == [[0, 0], [1, 1], [2, 2]][it] and st["round"] == it + 1

    # a resting partition is skipped by every stage
    hip.nnd_reverse_sample(*args)
    hip.nnd_local_join(*args)
    hip.nnd_merge(*args)
    hip.synchronize()
    rest = ws.read()
    for key in ("list_ids", "list_dists", "fwd_new", "fwd_old", "bloom", "offers", "rev_tables", "counts"):
        np.testing.assert_array_equal(rest[key], st[key], err_msg=key)

    # finalize: the `degree` nearest entries of the whole list by (distance, id) (the sub-lists merged by distance)
    d_knn = hip.DeviceArray((num, degree), np.uint32)
    hip.nnd_finalize(num, dim, d_ss, d_sl, 2, degree, d_knn, None, ws.buf, ws.bytes)
    hip.synchronize()
    knn = d_knn.numpy()
    for node in range(num):
        ent = sorted((int(np.float32(d).view(np.uint32)), int(v) & ~OLD) for v, d in zip(st["list_ids"][node], st["list_dists"][node]) if v != INV)
        want = [e[1] for e in ent[:degree]]
        assert knn[node, :len(want)].tolist() == want
    assert (knn < lim).all()


def test_crowded_offer_table_announces_a_threshold(hip):
    """A hub: thousands of offers for one node.  Built by hand: every list samples the same two points, so those receive
    offers from every join.  Whatever the order of arrival, every slot of the hub's table ends with the smallest key sent
    to it, the merge uses the 32 best of them, and the hub announces a distance threshold for the next join."""
    num, dim, degree = 10000, 128, 32
    rows = lowdim_data(num, dim, seed=9)
    seg_start, seg_len = np.array([0], np.uint32), np.array([num], np.uint32)
    d_rows = hip.DeviceArray.from_numpy(rows)
    d_ss, d_sl = hip.DeviceArray.from_numpy(seg_start), hip.DeviceArray.from_numpy(seg_len)
    ws = Workspace(hip, num, dim, degree)
    args = (num, dim, d_ss, d_sl, 1, degree, ws.buf, ws.bytes)
    hip.nnd_prepare(d_rows, num, dim, d_ss, d_sl, 1, degree, 1, ws.buf, ws.bytes)
    hip.synchronize()
    # every list's first two "new" samples become points 0 and 1 (the others stay random)
    w = ws.buf.numpy()
    fwd = w[ws.l.fwd_new // 4: ws.l.fwd_new // 4 + num * S].reshape(num, S)
    fwd[2:, 0] = 0
    fwd[2:, 1] = 1
    for r in range(2, num):        # keep a list's samples distinct
        for c in range(2, S):
            if fwd[r, c] in (0, 1):
                fwd[r, c] = 2 + (r + c) % (num - 2)
    ws.buf.upload(w)
    hip.nnd_local_join(*args)
    hip.synchronize()
    after = ws.read()
    offers = model_join(dict(after, fwd_new=fwd), rows, 0, num)
    assert len(offers[0]) > 4 * SLOTS and len(set(offers[0])) > 200          # thousands of arrivals, a few hundred distinct
    for t in (0, 1, 2, 500, 9999):
        np.testing.assert_array_equal(after["offers"][t], model_offer_table([offer_key(d, c) for d, c in offers.get(t, [])], 0))
    print("the hub holds", len(offers_held(after, 0)), "offers", flush=True)
    assert len(offers_held(after, 0)) >= 160 > len(offers_held(after, 2))
    hip.nnd_merge(*args)
    hip.synchronize()
    merged = ws.read()
    for node in (0, 1, 2, 500, 9999):
        l_ids, l_d, fn, fo, words, _ = model_merge(after, node, ws.l.width, ws.l.bloom_sets)
        np.testing.assert_array_equal(merged["list_ids"][node], l_ids)
        np.testing.assert_array_equal(merged["list_dists"][node], l_d)
        assert merged["fwd_new"][node, :len(fn)].tolist() == fn
    assert (merged["offers"] == NO_OFFER).all()
    # the hub has announced a threshold; a second join of the same lists sends it only what lies below
    thr = int(merged["offer_thr"][0])
    assert thr == model_offer_threshold(after, 0) == offers_held(after, 0)[63] >> 32
    assert int(merged["offer_thr"][2]) == INV
    w = ws.buf.numpy()
    w[ws.l.fwd_new // 4: ws.l.fwd_new // 4 + num * S] = fwd.reshape(-1)
    w[ws.l.counts // 4: ws.l.counts // 4 + num * 4].reshape(num, 4)[:] = after["counts"]
    ws.buf.upload(w)
    hip.nnd_local_join(*args)
    hip.synchronize()
    again = ws.read()
    below = [offer_key(d, c) for d, c in offers[0] if offer_key(d, c) >> 32 < thr]
    assert 0 < len(below) < len(offers[0])
    np.testing.assert_array_equal(again["offers"][0], model_offer_table(below, 0))
    assert offers_held(again, 0)[:S] == offers_held(after, 0)[:S]


@pytest.mark.parametrize("degree", [32, 64])
def test_sample_stage_on_its_own(hip, degree):
    """sample_graph (nn_descent.cuh:1040-1071) as a stage: on lists whose first 32 entries prepare has flagged, a second
    call draws the next 32 unflagged entries in storage order as new samples (all of a 32-wide list is flagged by then:
    none) and the first 32 flagged ones as old samples."""
    num, dim = 1200, 128
    rows = lowdim_data(num, dim, seed=17)
    seg_start, seg_len = np.array([0, 700], np.uint32), np.array([700, 500], np.uint32)
    d_rows = hip.DeviceArray.from_numpy(rows)
    d_ss, d_sl = hip.DeviceArray.from_numpy(seg_start), hip.DeviceArray.from_numpy(seg_len)
    ws = Workspace(hip, num, dim, degree)
    args = (num, dim, d_ss, d_sl, 2, degree, ws.buf, ws.bytes)
    hip.nnd_prepare(d_rows, num, dim, d_ss, d_sl, 2, degree, 4, ws.buf, ws.bytes)
    hip.synchronize()
    before = ws.read()
    hip.nnd_sample(*args)
    hip.synchronize()
    after = ws.read()
    width = ws.l.width
    for node in range(num):
        row = before["list_ids"][node]
        unflagged = [int(v) for v in row if v != INV and not v & OLD][:S]
        flagged = [int(v) & ~OLD for v in row if v != INV and v & OLD][:S]
        assert after["counts"][node].tolist() == [len(unflagged), len(flagged), 0, 0]
        assert after["fwd_new"][node, :len(unflagged)].tolist() == unflagged
        assert after["fwd_old"][node, :len(flagged)].tolist() == flagged
        want = row.copy()
        taken = 0
        for j in range(width):
            if want[j] != INV and not want[j] & OLD and taken < S:
                want[j] |= np.uint32(OLD)
                taken += 1
        np.testing.assert_array_equal(after["list_ids"][node], want)
    assert (after["counts"][:, 0] == (0 if width == 32 else S)).all() and (after["counts"][:, 1] == S).all()


@pytest.mark.parametrize("degree", [32, 64])
def test_small_partitions_hold_no_id_twice(hip, degree):
    """Partitions with fewer points than list slots: the random start lists repeat ids (at distance FLT_MAX), and an offer
    for an id the list holds is rejected whatever distance the held copy carries (insert_to_ordered_list,
    nn_descent.cuh:916-943), so no list ever names a point twice."""
    num, dim = 400, 128
    rows = lowdim_data(num, dim, seed=31)
    seg_len = np.array([40, 20, 70, 270], dtype=np.uint32)
    seg_start = np.array([0, 40, 60, 130], dtype=np.uint32)
    d_rows = hip.DeviceArray.from_numpy(rows)
    d_ss, d_sl = hip.DeviceArray.from_numpy(seg_start), hip.DeviceArray.from_numpy(seg_len)
    ws = Workspace(hip, num, dim, degree)
    args = (num, dim, d_ss, d_sl, 4, degree, ws.buf, ws.bytes)
    hip.nnd_prepare(d_rows, num, dim, d_ss, d_sl, 4, degree, 5, ws.buf, ws.bytes)
    local = np.arange(num) - np.repeat(seg_start, seg_len)
    limit = np.repeat(seg_len, seg_len)
    for it in range(6):
        hip.nnd_reverse_sample(*args)
        hip.nnd_local_join(*args)
        hip.nnd_merge(*args)
        hip.synchronize()
        st = ws.read()
        for node in range(num):
            row = st["list_ids"][node]
            ids = (row[row != INV] & ~np.uint32(OLD)).tolist()
            assert len(set(ids)) == len(ids), (it, node)
            assert local[node] not in ids and all(i < limit[node] for i in ids)
    d_knn = hip.DeviceArray((num, degree), np.uint32)
    hip.nnd_finalize(num, dim, d_ss, d_sl, 4, degree, d_knn, None, ws.buf, ws.bytes)
    hip.synchronize()
    assert (d_knn.numpy() < limit[:, None]).all()


def fast_model_join(st, rows, seg_start, seg_len):
    """model_join with the arg-mins taken by numpy (first minimum = earlier position); also returns how many lists had
    (at most 32 new members, of those more than 32 old ones, more than 32 new members)."""
    offers, shapes = {}, [0, 0, 0]
    half = rows.astype(np.float16).astype(np.float32)
    norms = (rows.astype(np.float32) ** 2).sum(1, dtype=np.float32)
    for node in range(seg_start, seg_start + seg_len):
        c = st["counts"][node]
        new = _dedupe(st["fwd_new"][node, :c[0]], reverse_samples(st, node, 0), seg_len)
        old = _dedupe(st["fwd_old"][node, :c[1]], reverse_samples(st, node, 1), seg_len)
        if not new:
            continue
        shapes[0 if len(new) <= S else 2] += 1
        shapes[1] += len(new) <= S and len(old) > S
        new_a, old_a = np.array(new), np.array(old, dtype=np.int64)
        xn, nn_ = half[seg_start + new_a], norms[seg_start + new_a]
        d = np.maximum(nn_[:, None] + nn_[None, :] - 2.0 * (xn @ xn.T), 0.0).astype(np.float32)
        np.fill_diagonal(d, np.inf)
        if len(new) > 1:
            for i, j in enumerate(d.argmin(1)):
                offers.setdefault(new[i], []).append((float(d[i, j]), new[j]))
        if old:
            xo, no_ = half[seg_start + old_a], norms[seg_start + old_a]
            d = np.maximum(nn_[:, None] + no_[None, :] - 2.0 * (xn @ xo.T), 0.0).astype(np.float32)
            d[new_a[:, None] == old_a[None, :]] = np.inf        # a point in both lists is no partner of itself
            for i, j in enumerate(d.argmin(1)):
                if np.isfinite(d[i, j]):
                    offers.setdefault(new[i], []).append((float(d[i, j]), old[j]))
            for j, i in enumerate(d.argmin(0)):
                if np.isfinite(d[i, j]):
                    offers.setdefault(old[j], []).append((float(d[i, j]), new[i]))
    kept = {k: sorted(o for o in v if offer_key(*o) >> 32 < int(st["offer_thr"][seg_start + k])) for k, v in offers.items()}
    return kept, shapes


@pytest.mark.parametrize("dim", [40, 96, 128, 136])
def test_both_join_kernels_match_model(hip, dim):
    """Six rounds, so that lists with few new members (one wavefront each, rows of up to 128 dims) and lists with many (one
    workgroup each) both occur, with one and with two blocks of old members; row lengths that are no multiple of 16
    (the last matrix step half empty), below 128 and above it.  Every node's offer table must be the model's."""
    num, degree = 1800, 32
    rows = lowdim_data(num, dim, seed=11)
    # the last two partitions are hardly larger / smaller than a list: their start lists hold an id twice / are not full
    seg_start, seg_len = np.array([0, 1500, 1745, 1780], np.uint32), np.array([1500, 245, 35, 20], np.uint32)
    d_rows = hip.DeviceArray.from_numpy(rows)
    d_ss, d_sl = hip.DeviceArray.from_numpy(seg_start), hip.DeviceArray.from_numpy(seg_len)
    ws = Workspace(hip, num, dim, degree)
    args = (num, dim, d_ss, d_sl, 4, degree, ws.buf, ws.bytes)
    hip.nnd_prepare(d_rows, num, dim, d_ss, d_sl, 4, degree, 7, ws.buf, ws.bytes)
    seen = np.zeros(3, np.int64)
    for it in range(6):
        print("dim", dim, "round", it, flush=True)
        hip.nnd_reverse_sample(*args)
        hip.synchronize()
        st = ws.read()
        hip.nnd_local_join(*args)
        hip.synchronize()
        after = ws.read()
        for s0, l0 in zip(seg_start.tolist(), seg_len.tolist()):
            offers, shapes = fast_model_join(st, rows, s0, l0)
            seen += shapes
            for t in range(l0):
                exp = model_offer_table([offer_key(d, c) for d, c in offers.get(t, [])], it, ws.l.offer_slots)
                np.testing.assert_array_equal(after["offers"][s0 + t], exp, err_msg="round %d, offer table of node %d" % (it, s0 + t))
        hip.nnd_merge(*args)
        hip.nnd_converge(num, dim, d_ss, d_sl, 4, degree, 0.0, ws.buf, ws.bytes)
    print("lists with at most 32 new members %d (%d of them with more than 32 old ones), with more %d" % tuple(seen), flush=True)
    assert seen.min() > 0
