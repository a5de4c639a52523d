"""GPU NN-descent against exact kNN and the CPU restatement (statistical parity: graph recall)."""
import numpy as np
import pytest

from conftest import lowdim_data, lowdim_float_data

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from glide_amd import capi
    capi.set_device(0)
    return capi


def gpu_nnd(hip, rdata, seg_start, seg_len, k, iterations, seed=0, threshold=0.0):
    n, dim = rdata.shape
    d_data = hip.DeviceArray.from_numpy(rdata, np.float32)
    d_ss, d_sl = hip.DeviceArray.from_numpy(seg_start, np.uint32), hip.DeviceArray.from_numpy(seg_len, np.uint32)
    knn = hip.DeviceArray((n, k), np.uint32)
    wb = hip.nnd_workspace_bytes(n, dim, k)
    ws = hip.DeviceArray(wb // 16 + 1, np.dtype("V16"))
    stats = hip.DeviceArray.from_numpy(np.zeros(2, np.uint64))
    hip.nnd_build(d_data, n, dim, d_ss, d_sl, seg_start.size, k, iterations, threshold, seed, knn, ws, wb, stats)
    hip.synchronize()
    return knn.numpy(), stats.numpy()


def partition_recall(knn, rdata, seg_start, seg_len, k, sample=400, metric=0):
    from glide_amd.datasets import recall
    from oracle import oracle as O
    out = []
    for s, l in zip(seg_start.tolist(), seg_len.tolist()):
        if l <= k + 1:
            continue
        sub = rdata[s:s + l]
        m = min(sample, l)
        gt, _ = O.bruteforce_knn(sub, sub[:m], k, metric, exclude_self=True)
        out.append(recall(knn[s:s + m], gt, k))
    return float(np.mean(out))


def test_nnd_structure_and_recall(hip):
    from oracle import oracle as O
    data = lowdim_data(12000, 128, seed=21)
    seg_len = np.array([5000, 4000, 2990, 10], dtype=np.uint32)       # the last one stands in for a tiny boundary list
    seg_start = O.segment_starts(np.append(seg_len, 0))[:4]
    k = 32
    knn, stats = gpu_nnd(hip, data, seg_start, seg_len, k, 10)
    # structure: ids are partition-local, no self loops, no repeated neighbour in partitions larger than k
    for s, l in zip(seg_start.tolist(), seg_len.tolist()):
        rows = knn[s:s + l]
        assert (rows < l).all()
        if l > 4 * k:   # partitions with fewer points than slots are padded with pseudo-random ids, like the reference's shrink step
            assert (rows != np.arange(l, dtype=np.uint32)[:, None]).all()
            srt = np.sort(rows, axis=1)
            assert (np.diff(srt.astype(np.int64), axis=1) != 0).all()
    r_gpu = partition_recall(knn, data, seg_start, seg_len, k)
    cpu = O.nnd_build(data, seg_start, seg_len, k, 10).astype(np.uint32)
    r_cpu = partition_recall(cpu, data, seg_start, seg_len, k)
    print("graph recall@32 after 10 iterations: gpu %.4f cpu-restatement %.4f; offers %d, declined by their target's threshold %d" % (r_gpu, r_cpu, stats[0], stats[1]))
    assert r_gpu >= 0.95
    assert r_gpu >= r_cpu - 0.005      # within half a point of the reference algorithm at equal degree / iterations


def test_nnd_rows_are_sorted_by_distance(hip):
    from oracle import oracle as O
    data = lowdim_data(4000, 128, seed=22)
    seg_len = np.array([4000], dtype=np.uint32)
    seg_start = np.array([0], dtype=np.uint32)
    knn, _ = gpu_nnd(hip, data, seg_start, seg_len, 32, 12)
    d = np.sqrt(((data[knn[:200].astype(np.int64)] - data[:200, None, :]) ** 2).sum(-1))
    assert (np.diff(d, axis=1) >= -1e-3).all()       # ascending (fp16 tile distances; integer data is exact)


def test_nnd_k64_cosine_dim96(hip):
    from oracle import oracle as O
    data = lowdim_float_data(6000, 96, seed=23)
    seg_len = np.array([3500, 2500], dtype=np.uint32)
    seg_start = np.array([0, 3500], dtype=np.uint32)
    knn, _ = gpu_nnd(hip, data, seg_start, seg_len, 64, 12)
    assert knn.shape == (6000, 64)
    r = partition_recall(knn, data, seg_start, seg_len, 64, sample=200, metric=1)
    print("graph recall@64 (cosine, dim 96): %.4f" % r)
    assert r >= 0.93


@pytest.mark.parametrize("dim", [960, 2048, 4096])
def test_nnd_long_rows(hip, dim):
    """Rows of 960 dims and of the longest length the beam kernels take, against the CPU restatement."""
    from oracle import oracle as O
    rng = np.random.default_rng(5)
    base = rng.random((40, dim)).astype(np.float32)
    data = (base[rng.integers(0, 40, 3000)] + rng.random((3000, dim)).astype(np.float32) * 0.3).astype(np.float32)
    seg_len = np.array([3000], dtype=np.uint32)
    seg_start = np.array([0], dtype=np.uint32)
    knn, _ = gpu_nnd(hip, data, seg_start, seg_len, 32, 10)
    r = partition_recall(knn, data, seg_start, seg_len, 32, sample=200)
    cpu = O.nnd_build(data, seg_start, seg_len, 32, 10).astype(np.uint32)
    r_cpu = partition_recall(cpu, data, seg_start, seg_len, 32, sample=200)
    print("graph recall@32 (dim %d): gpu %.4f cpu-restatement %.4f" % (dim, r, r_cpu))
    assert r >= 0.85 and r >= r_cpu - 0.01


def test_nnd_termination_threshold(hip):
    """With the reference's default threshold both sides stop early, at about the same graph recall; the GPU run
    then costs fewer offers than the fixed-length run."""
    from oracle import oracle as O
    rdata = lowdim_data(30000, 128, seed=21)
    seg_start, seg_len = np.array([0, 18000], np.uint32), np.array([18000, 12000], np.uint32)
    full, st_full = gpu_nnd(hip, rdata, seg_start, seg_len, 32, 20)
    early, st_early = gpu_nnd(hip, rdata, seg_start, seg_len, 32, 20, threshold=1e-4)
    cpu = O.nnd_build(rdata, seg_start, seg_len, 32, 20, 0, termination_threshold=1e-4).astype(np.uint32)
    r_full, r_early, r_cpu = (partition_recall(k, rdata, seg_start, seg_len, 32) for k in (full, early, cpu))
    print("graph recall@32: 20 rounds %.4f, with threshold gpu %.4f cpu %.4f; offers %d vs %d" % (r_full, r_early, r_cpu, st_early[0], st_full[0]))
    assert st_early[0] < 0.8 * st_full[0]
    assert r_early >= r_cpu - 0.005 and r_early >= 0.98


def test_nnd_rejects_unsupported(hip):
    d = hip.DeviceArray(1024, np.float32)
    with pytest.raises(hip.GlideHipError) as e:
        hip.nnd_build(d, 8, 128, d, d, 1, 257, 1, 0.0, 0, d, d, 1 << 30)      # above the widest degree the build searches take
    assert e.value.code == -1
    with pytest.raises(hip.GlideHipError) as e:
        hip.nnd_build(d, 8, 128, d, d, 1, 32, 1, 0.0, 0, d, d, 16)      # workspace too small
    assert e.value.code == -2


@pytest.mark.parametrize("dim,k", [(4, 8), (36, 16), (100, 32), (132, 48), (260, 64), (1024, 24), (128, 96), (64, 128), (128, 160), (96, 256)])
def test_nnd_shapes(hip, dim, k):
    """Dimensions that are not a multiple of the 64-dim chunk of the join (or of 8) and list widths 32, 64, 96, 128, 192,
    224 and 352 (the reference accepts any degree, nn_descent.cuh:1423-1430; its evaluation runs degree 96; the build
    searches that read the kNN graph take degrees up to 256)."""
    data = lowdim_data(3000, dim, latent=min(8, dim), seed=dim)
    seg_len = np.array([1800, 1200], dtype=np.uint32)
    seg_start = np.array([0, 1800], dtype=np.uint32)
    knn, _ = gpu_nnd(hip, data, seg_start, seg_len, k, 12)
    for s, l in zip(seg_start.tolist(), seg_len.tolist()):
        rows = knn[s:s + l]
        assert (rows < l).all() and (rows != np.arange(l, dtype=np.uint32)[:, None]).all()
    r = partition_recall(knn, data, seg_start, seg_len, k, sample=200)
    print("graph recall@%d (dim %d): %.4f" % (k, dim, r))
    if k > 64:
        # at most 32 offers a round enter a list of 128 or 192 slots: after 12 rounds the tail is still filling, in
        # the CPU restatement alike; the bar is the restatement's recall at equal degree and iterations
        from oracle import oracle as O
        cpu = O.nnd_build(data, seg_start, seg_len, k, 12).astype(np.uint32)
        r_cpu = partition_recall(cpu, data, seg_start, seg_len, k, sample=200)
        print("cpu restatement: %.4f" % r_cpu)
        assert r >= r_cpu - 0.005
    else:
        assert r >= (0.9 if dim > 4 else 0.6)      # 4 small-integer dimensions are mostly ties


@pytest.mark.parametrize("k", [32, 64])
def test_nnd_recall_round_by_round(hip, k):
    """Graph recall@k after 2, 4, 6, 8 and 12 rounds against the CPU restatement at the same number of rounds, on the
    benchmark's mixture: the GPU lists have to fill at the reference algorithm's pace, not only end where it ends
    (with k = 64 the lists are three id-keyed sub-lists on both sides)."""
    from glide_amd import datasets as D
    from oracle import oracle as O
    data = D.gmm_clipped(16000, 128, seed=77)
    seg_len = np.array([9000, 7000], dtype=np.uint32)
    seg_start = np.array([0, 9000], dtype=np.uint32)
    seen = []
    for rounds in (2, 4, 6, 8, 12):
        r_gpu = r_cpu = 0.0
        for seed in (3, 4):          # the two sides draw different random start lists: two seeds a side, 3 000 rows scored
            knn, _ = gpu_nnd(hip, data, seg_start, seg_len, k, rounds, seed=seed)
            cpu = O.nnd_build(data, seg_start, seg_len, k, rounds, seed=seed).astype(np.uint32)
            r_gpu += partition_recall(knn, data, seg_start, seg_len, k, sample=1500) / 2
            r_cpu += partition_recall(cpu, data, seg_start, seg_len, k, sample=1500) / 2
        print("k %d, %2d rounds: graph recall@%d gpu %.4f cpu-restatement %.4f" % (k, rounds, k, r_gpu, r_cpu), flush=True)
        seen.append((rounds, r_gpu, r_cpu))
    # Half a point from the sixth round on; three quarters of a point in the first rounds, where recall rises by ten
    # points a round and the few offers that lose both their slots to nearer candidates show as a fortieth of a round.
    for rounds, r_gpu, r_cpu in seen:
        assert r_gpu >= r_cpu - (0.0075 if rounds < 6 else 0.005) and r_gpu <= r_cpu + 0.03, (k, seen)


def test_nnd_same_seed_same_graph(hip):
    """Nothing in the build depends on the order in which atomic operations arrive: the offer tables keep the smallest
    keys, the reverse tables the smallest sources, and both are sorted before use.  Mixture data, where a few points
    receive thousands of offers per round, and a degree with three sub-lists."""
    from glide_amd import datasets as D
    data = D.gmm_clipped(24000, 128, seed=7)
    seg_start, seg_len = np.array([0, 14000], np.uint32), np.array([14000, 10000], np.uint32)
    for k, rounds in ((32, 6), (64, 4)):
        a, st_a = gpu_nnd(hip, data, seg_start, seg_len, k, rounds, seed=3)
        b, st_b = gpu_nnd(hip, data, seg_start, seg_len, k, rounds, seed=3)
        c, _ = gpu_nnd(hip, data, seg_start, seg_len, k, rounds, seed=4)
        # st[0]: distinct offers the merge steps found in the tables; st[1]: offers a join did not send because they were not
        # below the threshold their target had announced.  A join decides that per offer from values fixed before the round
        # starts, so both counts repeat with the graph
        assert np.array_equal(a, b) and st_a[0] == st_b[0] and st_a[1] == st_b[1]
        assert not np.array_equal(a, c)
        print("degree %d: offers merged %d, declined by a target's threshold %d" % (k, st_a[0], st_a[1]))


@pytest.mark.parametrize("k,dim", [(32, 128), (64, 96), (32, 200)])
def test_nnd_build_equals_its_stages(hip, k, dim):
    """glide_hip_nnd_build takes shortcuts its stage entry points do not: the merge kernel scatters the next round's
    reverse samples itself, from the fourth round on the workgroup join takes runs of 16 lists per workgroup,
    and from the fifth the joins no longer read a slot before sending to it.  None of this may show: eight rounds run
    stage by stage must end in the very graph the fused build gives (dims with and without the one-wavefront join)."""
    from glide_amd import datasets as D
    data = D.gmm_clipped(12000, dim, seed=21)
    seg_start, seg_len = np.array([0, 7000], np.uint32), np.array([7000, 5000], np.uint32)
    rounds, seed = 8, 5
    fused, _ = gpu_nnd(hip, data, seg_start, seg_len, k, rounds, seed=seed)
    n = data.shape[0]
    d_data = hip.DeviceArray.from_numpy(data, np.float32)
    d_ss, d_sl = hip.DeviceArray.from_numpy(seg_start, np.uint32), hip.DeviceArray.from_numpy(seg_len, np.uint32)
    wb = hip.nnd_workspace_bytes(n, dim, k)
    ws = hip.DeviceArray(wb // 16 + 1, np.dtype("V16"))
    args = (n, dim, d_ss, d_sl, 2, k, ws, wb)
    hip.nnd_prepare(d_data, n, dim, d_ss, d_sl, 2, k, seed, ws, wb)
    for _ in range(rounds):
        hip.nnd_reverse_sample(*args)
        hip.nnd_local_join(*args)
        hip.nnd_merge(*args)
        hip.nnd_converge(n, dim, d_ss, d_sl, 2, k, 0.0, ws, wb)
    knn = hip.DeviceArray((n, k), np.uint32)
    hip.nnd_finalize(n, dim, d_ss, d_sl, 2, k, knn, None, ws, wb)
    hip.synchronize()
    assert np.array_equal(knn.numpy(), fused)
