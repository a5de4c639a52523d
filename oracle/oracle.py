"""ctypes binding of the CPU oracle (oracle/libglide_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg.
The product (glide_amd) never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libglide_oracle.so")
_lib = None

EUCLIDEAN, COSINE = 0, 1
INVALID = 0xFFFFFFFF


def build(force=False):
    """Compile the oracle with g++ (make).  Building the checker is not using it."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)


class Stats(C.Structure):
    _fields_ = [("iterations", C.c_uint64), ("rows_scored", C.c_uint64), ("graph_rows", C.c_uint64)]

    def as_dict(self):
        return {"iterations": self.iterations, "rows_scored": self.rows_scored, "graph_rows": self.graph_rows}


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.go_distance.restype = C.c_float
        for name in ("go_hash_bitlen", "go_hash_reset_interval", "go_nnd_extended_degree", "go_xorshift32",
                     "go_max_candidate", "go_max_beam", "go_max_centroid_search", "go_max_centroid_partition",
                     "go_prune"):
            getattr(_lib, name).restype = C.c_uint32
    return _lib


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _u32(a):
    return np.ascontiguousarray(a, dtype=np.uint32)


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


u32 = C.c_uint32
f32 = C.c_float


# ------------------------------------------------------------------ params
def hash_bitlen(beam, degree, fill=0.5, min_bitlen=0):
    return lib().go_hash_bitlen(u32(beam), u32(degree), f32(fill), u32(min_bitlen))


def hash_reset_interval(beam, degree, fill, bitlen):
    return lib().go_hash_reset_interval(u32(beam), u32(degree), f32(fill), u32(bitlen))


def adjust_search_params(min_iterations, max_iterations, beam):
    mi, b = u32(max_iterations), u32(beam)
    lib().go_adjust_search_params(u32(min_iterations), C.byref(mi), C.byref(b))
    return mi.value, b.value


def search_params(beam, degree, fill=0.5):
    """SearchParameter sizing as the reference mains do it (small_search.cu:102-108)."""
    max_iter, beam = adjust_search_params(0, 0, beam)
    hb = hash_bitlen(beam, degree, fill, 0)
    reset = hash_reset_interval(beam, degree, fill, hb)
    return dict(beam=beam, max_iterations=max_iter, min_iterations=0, hash_bit=hb, hash_reset_interval=reset)


def nnd_extended_degree(k):
    return lib().go_nnd_extended_degree(u32(k))


def xorshift32(x):
    return lib().go_xorshift32(u32(x))


# ------------------------------------------------------------------ primitives
def bitonic_warp_sort(keys, vals):
    k, v = _f32(keys).copy(), _u32(vals).copy()
    assert lib().go_bitonic_warp_sort(_p(k), _p(v), u32(k.size)) == 0
    return k, v


def bitonic_warp_merge(keys, vals, rng):
    k, v = _f32(keys).copy(), _u32(vals).copy()
    assert lib().go_bitonic_warp_merge(_p(k), _p(v), u32(k.size), u32(rng)) == 0
    return k, v


def sort_with_key_value(max_number, vals, keys):
    k, v = _f32(keys).copy(), _u32(vals).copy()
    assert lib().go_sort_with_key_value(u32(max_number), u32(k.size), _p(v), _p(k)) == 0
    return v, k


def sort_for_candidate(max_cand, cand_dist, cand_id, degree, beam):
    d, i = _f32(cand_dist).copy(), _u32(cand_id).copy()
    assert lib().go_sort_for_candidate(u32(max_cand), _p(d), _p(i), u32(degree), u32(beam)) == 0
    return d, i


def sort_for_beam(max_beam, beam_dist, beam_id, beam, cand_dist, cand_id, degree, first):
    bd, bi = _f32(beam_dist).copy(), _u32(beam_id).copy()
    cd, ci = _f32(cand_dist), _u32(cand_id)
    assert lib().go_sort_for_beam(u32(max_beam), _p(bd), _p(bi), u32(beam), _p(cd), _p(ci), u32(degree),
                                  C.c_int(int(first))) == 0
    return bd, bi


def hashmap_insert_seq(bitlen, keys, table=None):
    keys = _u32(keys)
    if table is None:
        table = np.empty(1 << bitlen, dtype=np.uint32)
        lib().go_hashmap_init(_p(table), u32(bitlen))
    flags = np.empty(keys.size, dtype=np.uint32)
    lib().go_hashmap_insert_seq(_p(table), u32(bitlen), _p(keys), u32(keys.size), _p(flags))
    return flags, table


def distance(a, b, metric=EUCLIDEAN):
    a, b = _f32(a), _f32(b)
    return float(lib().go_distance(_p(a), _p(b), u32(a.size), C.c_int(metric)))


def distance_batch(a, b, metric=EUCLIDEAN):
    a, b = _f32(a), _f32(b)
    return np.array([distance(a[i], b[i], metric) for i in range(a.shape[0])], dtype=np.float32)


# ------------------------------------------------------------------ pipeline stages
def search(data, graph, centroids, start_points, queries, top_k, beam, max_iterations, min_iterations, hash_bit,
           hash_reset_interval, metric=EUCLIDEAN, threads=0):
    data, graph, centroids, queries = _f32(data), _u32(graph), _f32(centroids), _f32(queries)
    start_points = _u32(start_points)
    nq = queries.shape[0]
    ids = np.empty((nq, top_k), dtype=np.uint32)
    dists = np.empty((nq, top_k), dtype=np.float32)
    st = Stats()
    rc = lib().go_search(_p(data), u32(data.shape[0]), u32(data.shape[1]), _p(graph), u32(graph.shape[1]),
                         _p(centroids), u32(centroids.shape[0]), _p(start_points), _p(queries), u32(nq), u32(top_k),
                         u32(beam), u32(max_iterations), u32(min_iterations), u32(hash_bit),
                         u32(hash_reset_interval), C.c_int(metric), _p(ids), _p(dists), C.byref(st),
                         C.c_int(threads))
    if rc != 0:
        raise ValueError("oracle search: unsupported parameters")
    return ids, dists, st.as_dict()


def partition_assign(data, centroids, boundary_factor, metric=EUCLIDEAN, threads=0):
    data, centroids = _f32(data), _f32(centroids)
    n, c = data.shape[0], centroids.shape[0]
    seg_idx = np.empty((n, 3), dtype=np.uint32)
    seg_len = np.empty(c + 1, dtype=np.uint32)
    nearest = np.empty((n, 2), dtype=np.float32)
    rc = lib().go_partition_assign(_p(data), u32(n), u32(data.shape[1]), _p(centroids), u32(c), f32(boundary_factor),
                                   C.c_int(metric), _p(seg_idx), _p(seg_len), _p(nearest), C.c_int(threads))
    if rc != 0:
        raise ValueError("oracle partition_assign: unsupported parameters")
    return seg_idx, seg_len, nearest


def segment_starts(seg_len):
    return np.concatenate([[0], np.cumsum(seg_len[:-1], dtype=np.uint64)]).astype(np.uint32)


def reorder(data, seg_idx, seg_start, reorder_num):
    data, seg_idx, seg_start = _f32(data), _u32(seg_idx), _u32(seg_start)
    out = np.empty((reorder_num, data.shape[1]), dtype=np.float32)
    mp = np.empty(reorder_num, dtype=np.uint32)
    lib().go_reorder(_p(data), u32(data.shape[0]), u32(data.shape[1]), _p(seg_idx), _p(seg_start), _p(out), _p(mp))
    return out, mp


def build_subgraph(reorder_data, num, knn_graph, mp, seg_start, seg_len, start_points, graph_degree, sp, relaxant,
                   metric=EUCLIDEAN, graph=None, threads=0):
    reorder_data, knn_graph, mp = _f32(reorder_data), _u32(knn_graph), _u32(mp)
    seg_start, seg_len, start_points = _u32(seg_start), _u32(seg_len), _u32(start_points)
    if graph is None:
        graph = np.full((num, graph_degree), INVALID, dtype=np.uint32)
    st = Stats()
    rc = lib().go_build_subgraph(_p(reorder_data), u32(num), u32(reorder_data.shape[1]), _p(knn_graph),
                                 u32(knn_graph.shape[1]), _p(mp), _p(seg_start), _p(seg_len), u32(seg_start.size),
                                 _p(start_points), u32(graph_degree), u32(sp["beam"]), u32(sp["max_iterations"]),
                                 u32(sp["min_iterations"]), u32(sp["hash_bit"]), u32(sp["hash_reset_interval"]),
                                 f32(relaxant), C.c_int(metric), _p(graph), C.byref(st), C.c_int(threads))
    if rc != 0:
        raise ValueError("oracle build_subgraph: unsupported parameters")
    return graph, st.as_dict()


def build_boundary(reorder_data, num, knn_graph, mp, start_point, graph, sp, relaxant, metric=EUCLIDEAN, threads=0):
    reorder_data, knn_graph, mp = _f32(reorder_data), _u32(knn_graph), _u32(mp)
    assert graph.dtype == np.uint32 and graph.flags.c_contiguous
    st = Stats()
    rc = lib().go_build_boundary(_p(reorder_data), u32(num), u32(reorder_data.shape[0]), u32(reorder_data.shape[1]),
                                 _p(knn_graph), u32(knn_graph.shape[1]), _p(mp), u32(start_point),
                                 u32(graph.shape[1]), u32(sp["beam"]), u32(sp["max_iterations"]),
                                 u32(sp["min_iterations"]), u32(sp["hash_bit"]), u32(sp["hash_reset_interval"]),
                                 f32(relaxant), C.c_int(metric), _p(graph), C.byref(st), C.c_int(threads))
    if rc != 0:
        raise ValueError("oracle build_boundary: unsupported parameters")
    return graph, st.as_dict()


def merge_boundary_row(row, neighbors, mp):
    row, neighbors, mp = _u32(row).copy(), _u32(neighbors), _u32(mp)
    pad = np.full(((row.size + 31) // 32) * 32, INVALID, dtype=np.uint32)
    pad[:neighbors.size] = neighbors
    lib().go_merge_boundary_row(_p(row), u32(row.size), _p(pad), _p(mp))
    return row


def prune(data, segment_start, pool_ids, pool_dists, graph_degree, relaxant, metric=EUCLIDEAN):
    data, ids, ds = _f32(data), _u32(pool_ids).copy(), _f32(pool_dists).copy()
    nb = np.empty(((graph_degree + 31) // 32) * 32, dtype=np.uint32)
    n = lib().go_prune(_p(data), u32(data.shape[1]), u32(segment_start), _p(ids), _p(ds), u32(ids.size),
                       u32(graph_degree), f32(relaxant), C.c_int(metric), _p(nb))
    return nb[:graph_degree].copy(), int(n)


def reverse_edges(graph):
    g = _u32(graph).copy()
    lib().go_reverse_edges(_p(g), u32(g.shape[0]), u32(g.shape[1]))
    return g


def refine(data, graph, centroids, start_points, sp, relaxant, metric=EUCLIDEAN, threads=0):
    data, centroids, start_points = _f32(data), _f32(centroids), _u32(start_points)
    g = _u32(graph).copy()
    st = Stats()
    rc = lib().go_refine(_p(data), u32(data.shape[0]), u32(data.shape[1]), _p(g), u32(g.shape[1]), _p(centroids),
                         u32(centroids.shape[0]), _p(start_points), u32(sp["beam"]), u32(sp["max_iterations"]),
                         u32(sp["min_iterations"]), u32(sp["hash_bit"]), u32(sp["hash_reset_interval"]),
                         f32(relaxant), C.c_int(metric), C.byref(st), C.c_int(threads))
    if rc != 0:
        raise ValueError("oracle refine: unsupported parameters")
    return g, st.as_dict()


def select_segments(queries, centroids, min_segment_num, boundary_factor, metric=EUCLIDEAN):
    queries, centroids = _f32(queries), _f32(centroids)
    out = np.empty((queries.shape[0], centroids.shape[0]), dtype=np.uint32)
    rc = lib().go_select_segments(_p(queries), u32(queries.shape[0]), u32(queries.shape[1]), _p(centroids),
                                  u32(centroids.shape[0]), u32(min_segment_num), f32(boundary_factor), C.c_int(metric), _p(out))
    if rc != 0:
        raise ValueError("oracle select_segments: unsupported parameters")
    return out


def search_sub(seg_data, seg_graph, seg_map, queries, segment_ids, segment_id, start_point, top_k, sp, final_ids, final_dists,
               metric=EUCLIDEAN, threads=0):
    seg_data, seg_graph, seg_map, queries = _f32(seg_data), _u32(seg_graph), _u32(seg_map), _f32(queries)
    segment_ids = _u32(segment_ids)
    assert final_ids.dtype == np.uint32 and final_dists.dtype == np.float32
    st = Stats()
    rc = lib().go_search_sub(_p(seg_data), u32(seg_data.shape[1]), _p(seg_graph), u32(seg_graph.shape[1]), _p(seg_map), _p(queries),
                             u32(queries.shape[0]), _p(segment_ids), u32(segment_ids.shape[1]), u32(segment_id), u32(start_point),
                             u32(top_k), u32(sp["beam"]), u32(sp["max_iterations"]), u32(sp["min_iterations"]), u32(sp["hash_bit"]),
                             u32(sp["hash_reset_interval"]), C.c_int(metric), _p(final_ids), _p(final_dists), C.byref(st),
                             C.c_int(threads))
    if rc != 0:
        raise ValueError("oracle search_sub: unsupported parameters")
    return st.as_dict()


def build_segment(seg_data, knn_graph, start_point, graph_degree, sp, relaxant, metric=EUCLIDEAN, threads=0):
    seg_data, knn_graph = _f32(seg_data), _u32(knn_graph)
    graph = np.empty((seg_data.shape[0], graph_degree), dtype=np.uint32)
    st = Stats()
    rc = lib().go_build_segment(_p(seg_data), u32(seg_data.shape[0]), u32(seg_data.shape[1]), _p(knn_graph), u32(knn_graph.shape[1]),
                                u32(start_point), u32(graph_degree), u32(sp["beam"]), u32(sp["max_iterations"]),
                                u32(sp["min_iterations"]), u32(sp["hash_bit"]), u32(sp["hash_reset_interval"]), f32(relaxant),
                                C.c_int(metric), _p(graph), C.byref(st), C.c_int(threads))
    if rc != 0:
        raise ValueError("oracle build_segment: unsupported parameters")
    return graph, st.as_dict()


def refine_segment(seg_data, graph, start_point, sp, relaxant, metric=EUCLIDEAN, threads=0):
    seg_data = _f32(seg_data)
    g = _u32(graph).copy()
    st = Stats()
    rc = lib().go_refine_segment(_p(seg_data), u32(seg_data.shape[0]), u32(seg_data.shape[1]), _p(g), u32(g.shape[1]),
                                 u32(start_point), u32(sp["beam"]), u32(sp["max_iterations"]), u32(sp["min_iterations"]),
                                 u32(sp["hash_bit"]), u32(sp["hash_reset_interval"]), f32(relaxant), C.c_int(metric), C.byref(st),
                                 C.c_int(threads))
    if rc != 0:
        raise ValueError("oracle refine_segment: unsupported parameters")
    return g, st.as_dict()


def nnd_build(reorder_data, seg_start, seg_len, knn_degree, iterations, seed=0, threads=0, termination_threshold=0.0, shipped_loop=False):
    """termination_threshold = 0 runs exactly `iterations` rounds; the reference's default is 1e-4 (params.cuh:21).
    shipped_loop: the host loop as the reference ships it (partitions whose first row is not below their length get two
    rounds, no merge across sub-lists) instead of the intended algorithm."""
    reorder_data, seg_start, seg_len = _f32(reorder_data), _u32(seg_start), _u32(seg_len)
    out = np.empty((reorder_data.shape[0], knn_degree), dtype=np.int32)
    rc = (lib().go_nnd_build_shipped if shipped_loop else lib().go_nnd_build_ex)(_p(reorder_data), u32(reorder_data.shape[0]), u32(reorder_data.shape[1]), _p(seg_start),
                               _p(seg_len), u32(seg_start.size), u32(knn_degree), u32(iterations),
                               C.c_float(termination_threshold), u32(seed), _p(out), C.c_int(threads))
    if rc != 0:
        raise ValueError("oracle nnd_build failed: %d" % rc)
    return out


def nnd_build_from(reorder_data, seg_start, seg_len, knn_degree, iterations, start_lists, threads=0, termination_threshold=0.0):
    """nnd_build from the caller's start lists: (rows, extended degree) int32 partition-local ids, a row's sub-lists one
    after the other (sub-list s holds ids with id % num_sub == s), negative = empty slot."""
    reorder_data, seg_start, seg_len = _f32(reorder_data), _u32(seg_start), _u32(seg_len)
    start_lists = np.ascontiguousarray(start_lists, dtype=np.int32)
    assert start_lists.shape == (reorder_data.shape[0], nnd_extended_degree(knn_degree))
    out = np.empty((reorder_data.shape[0], knn_degree), dtype=np.int32)
    rc = lib().go_nnd_build_from(_p(reorder_data), u32(reorder_data.shape[0]), u32(reorder_data.shape[1]), _p(seg_start), _p(seg_len),
                                 u32(seg_start.size), u32(knn_degree), u32(iterations), C.c_float(termination_threshold),
                                 start_lists.ctypes.data_as(C.c_void_p), _p(out), C.c_int(threads))
    if rc != 0:
        raise ValueError("oracle nnd_build_from failed: %d" % rc)
    return out


def bruteforce_knn(data, queries, k, metric=EUCLIDEAN, exclude_self=False, threads=0):
    data, queries = _f32(data), _f32(queries)
    ids = np.empty((queries.shape[0], k), dtype=np.uint32)
    dists = np.empty((queries.shape[0], k), dtype=np.float32)
    lib().go_bruteforce_knn(_p(data), u32(data.shape[0]), u32(data.shape[1]), _p(queries), u32(queries.shape[0]),
                            u32(k), C.c_int(metric), C.c_int(int(exclude_self)), _p(ids), _p(dists), C.c_int(threads))
    return ids, dists


def kmeans(sample, k, iterations=20, seed=7):
    sample = _f32(sample)
    cent = np.empty((k, sample.shape[1]), dtype=np.float32)
    lib().go_kmeans(_p(sample), u32(sample.shape[0]), u32(sample.shape[1]), u32(k), u32(iterations), u32(seed),
                    _p(cent))
    return cent


def kmeans_seed(sample, k, seed=7):
    """k-means++ seeding with the HIP library's draws; returns (centroids, chosen sample rows)."""
    sample = _f32(sample)
    cent = np.empty((k, sample.shape[1]), dtype=np.float32)
    chosen = np.empty(k, dtype=np.uint32)
    lib().go_kmeans_seed(_p(sample), u32(sample.shape[0]), u32(sample.shape[1]), u32(k), u32(seed), _p(cent), _p(chosen))
    return cent, chosen


def kmeans_from(sample, centroids, iterations=20):
    sample, cent = _f32(sample), _f32(centroids).copy()
    lib().go_kmeans_from(_p(sample), u32(sample.shape[0]), u32(sample.shape[1]), u32(cent.shape[0]), u32(iterations), _p(cent))
    return cent


def build_index(data, centroid_num, graph_degree=32, knn_degree=32, boundary_factor=1.04, relaxant=1.05,
                build_beam=64, refine_beam=128, nnd_iterations=8, metric=EUCLIDEAN, seed=11, sample_factor=0.01,
                centroids=None, threads=0):
    """Whole small-build pipeline on the CPU (small_preprocess -> small_knn -> small_build); returns a dict."""
    data = _f32(data)
    n = data.shape[0]
    rng = np.random.default_rng(seed)
    if centroids is None:
        ns = max(int(n * sample_factor), centroid_num * 8)
        sample = data[rng.permutation(n)[:min(ns, n)]]
        centroids = kmeans(sample, centroid_num)
    seg_idx, seg_len, _ = partition_assign(data, centroids, boundary_factor, metric, threads)
    seg_start = segment_starts(seg_len)
    reorder_num = n + int(seg_len[centroid_num])
    rdata, mp = reorder(data, seg_idx, seg_start, reorder_num)
    knn = nnd_build(rdata, seg_start, seg_len, knn_degree, nnd_iterations, 0, threads).astype(np.uint32)
    local_sp = np.array([rng.integers(0, max(int(l), 1)) for l in seg_len], dtype=np.uint32)
    sp_build = search_params(build_beam, knn_degree)
    graph, st_build = build_subgraph(rdata, n, knn, mp, seg_start, seg_len, local_sp, graph_degree, sp_build,
                                     relaxant, metric, threads=threads)
    if reorder_num > n:
        graph, _ = build_boundary(rdata, n, knn, mp, int(local_sp[centroid_num]), graph, sp_build, relaxant, metric,
                                  threads=threads)
    start_points = mp[seg_start[:centroid_num] + local_sp[:centroid_num]].astype(np.uint32)
    graph = reverse_edges(graph)
    if refine_beam:
        sp_ref = search_params(refine_beam, knn_degree)   # small_build.cu:76-82 sizes the refine hash with knn_degree
        graph, _ = refine(data, graph, centroids, start_points, sp_ref, relaxant, metric, threads)
    return dict(centroids=centroids, seg_idx=seg_idx, seg_len=seg_len, seg_start=seg_start, reorder_data=rdata,
                map=mp, knn=knn, local_start_points=local_sp, start_points=start_points, graph=graph)
