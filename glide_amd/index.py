"""Host-side mirror of the reference's build/search interface on top of the C ABI.

Names, argument meaning and error behaviour follow the reference's C++ host layer:
  params.cuh           -> Metric, PartitionParameter, NNDescentParameter, IndexParameter, SearchParameter,
                          calculate_hash_bitlen, calculate_hash_reset_interval, adjust_search_params
  partition.cuh:159    -> preprocess()
  nn_descent.cuh:1405  -> build_nnd()
  glide.cuh:14-125     -> class GLIDE (ctor, load, build, search, accessors)
All device work goes through glide_amd.capi (libglide_hip.so); nothing here computes on the CPU beyond the
integer parameter arithmetic and the random choices the reference also makes on the host.
"""
import math
import time
from dataclasses import dataclass

import numpy as np

from . import capi

INVALID = 0xFFFFFFFF


class Metric:
    Euclidean = capi.EUCLIDEAN
    Cosine = capi.COSINE


@dataclass
class PartitionParameter:          # params.cuh:10-15
    centroid_num: int = 10
    boundary_factor: float = 1.05
    sample_factor: float = 0.01
    metric: int = Metric.Euclidean
    kmeans_iterations: int = 20     # cuVS kmeans is replaced by greedy k-means++ seeding + Lloyd steps; count and seed are explicit here
    seed: int = 7


@dataclass
class NNDescentParameter:          # params.cuh:17-25
    graph_degree: int = 64
    intermediate_graph_degree: int = 0
    max_iterations: int = 20
    termination_threshold: float = 0.0001
    seed: int = 0

    def __post_init__(self):
        if not self.intermediate_graph_degree:
            self.intermediate_graph_degree = int(1.5 * self.graph_degree)


@dataclass
class IndexParameter:              # params.cuh:27-35
    graph_degree: int = 32
    knn_degree: int = 32
    relaxant_factor: float = 1.05
    metric: int = Metric.Euclidean
    seed: int = 11                  # the reference draws start points from std::random_device


@dataclass
class SearchParameter:             # params.cuh:37-47
    top_k: int = 10
    beam: int = 100
    max_iterations: int = 0
    min_iterations: int = 0
    hash_bit: int = 0
    hash_max_fill_rate: float = 0.5
    hashmap_min_bitlen: int = 0
    hash_reset_interval: int = 1
    search_block_size: int = 0


def calculate_hash_bitlen(beam, graph_degree, hashmap_max_fill_rate, hashmap_min_bitlen):   # params.cuh:49-66
    max_visited_nodes = beam + graph_degree
    min_bitlen, max_bitlen = 8, 13
    if min_bitlen < hashmap_min_bitlen:
        min_bitlen = hashmap_min_bitlen
    hash_bitlen = min_bitlen
    fill = np.float32(hashmap_max_fill_rate)
    while max_visited_nodes > np.float32(1 << hash_bitlen) * fill:
        hash_bitlen += 1
    return min(hash_bitlen, max_bitlen)


def calculate_hash_reset_interval(beam, graph_degree, hashmap_max_fill_rate, hash_bitlen):  # params.cuh:68-80
    interval = 1
    fill = np.float32(hashmap_max_fill_rate)
    while True:
        if beam + graph_degree * (interval + 1) > np.float32(1 << hash_bitlen) * fill:
            break
        interval += 1
    return interval


def adjust_search_params(min_iterations, max_iterations, beam):                            # params.cuh:82-99
    """Returns (max_iterations, beam)."""
    m = max_iterations
    if max_iterations == 0:
        m = int(1 + min(beam * 1.1, beam + 10.0))
    if max_iterations < min_iterations:
        m = min_iterations
    if max_iterations < m:
        max_iterations = m
    if beam % 32:
        beam += 32 - (beam % 32)
    return max_iterations, beam


def make_search_parameter(beam, degree, top_k=10):
    """SearchParameter sized the way the reference mains do (small_search.cu:102-108, small_build.cu:61-82)."""
    p = SearchParameter(top_k=top_k, beam=beam)
    p.max_iterations, p.beam = adjust_search_params(p.min_iterations, p.max_iterations, p.beam)
    p.hash_bit = calculate_hash_bitlen(p.beam, degree, p.hash_max_fill_rate, p.hashmap_min_bitlen)
    p.hash_reset_interval = calculate_hash_reset_interval(p.beam, degree, p.hash_max_fill_rate, p.hash_bit)
    return p


def _check_sizes(beam, degree):
    # kernel_config.cuh:48,60: std::invalid_argument("Unsupported beam" / "Unsupported graph_degree")
    if beam > 512 or (beam > 256 and beam % 16):     # the second: adjust_search_params rounds beams to multiples of 32
        raise ValueError("Unsupported beam")
    if degree > 256:
        raise ValueError("Unsupported graph_degree")


class _Timer:
    """GPU seconds between two events on the default stream (the reference sums cudaEvent intervals)."""

    def __init__(self):
        self.start, self.stop = capi.Event(), capi.Event()

    def __enter__(self):
        self.start.record()
        return self

    def __exit__(self, *exc):
        self.stop.record()
        self.seconds = self.start.elapsed_ms(self.stop) / 1000.0


def pad_rows(rows, multiple=4):
    """Points as the entry points want them: fp32 rows on the device whose length is a multiple of four values.  The
    reference's kernels loop over single values and take any dim (distance.cuh:9-27); here rows are read in 16-byte
    pieces, so points of another length get zeros behind them once, which changes no squared distance, inner product
    or norm.  numpy (num, dim) or DeviceArray in, DeviceArray (num, padded dim) out -- the same DeviceArray when its
    rows already fit, else a padded copy made on the device."""
    d = rows if isinstance(rows, capi.DeviceArray) else capi.DeviceArray.from_numpy(rows, np.float32)
    num, dim = d.shape
    held = (dim + multiple - 1) // multiple * multiple
    if held == dim:
        return d
    out = capi.DeviceArray((num, held), np.float32)
    capi.copy_rows(d, num, dim, out, held)
    capi.synchronize()
    if d is not rows:
        d.free()
    return out


def cut_rows(d_rows, dim):
    """The first `dim` values of every row of a DeviceArray of points, as numpy: centroids or reordered rows of padded
    points in the length the caller's data has."""
    num, held = d_rows.shape
    if held == dim:
        return d_rows.numpy()
    out = capi.DeviceArray((num, dim), np.float32)
    capi.copy_rows(d_rows, num, held, out, dim)
    capi.synchronize()
    h = out.numpy()
    out.free()
    return h


def preprocess(param, d_data, result=None):
    """partition.cuh:159-193.  d_data: DeviceArray (num, dim) float32; rows of a length that is no multiple of four are
    padded (pad_rows), and the reordered rows and centroids returned then have the padded length (cut_rows gives them
    back in the data's own).

    Returns (d_reorder_data, d_map, h_segment_start, h_segment_length, d_centroids).  h_segment_* have
    centroid_num + 1 entries, the last being the boundary segment (start = num).
    """
    d_data = pad_rows(d_data)
    num, dim = d_data.shape
    c = param.centroid_num
    times = {}
    # get_centroids (partition.cuh:10-59): shuffle, sample, k-means on the sample
    sample_num = max(int(num * param.sample_factor), min(num, c))
    rng = np.random.default_rng(param.seed)
    ids = rng.permutation(num)[:sample_num].astype(np.uint32)
    d_ids = capi.DeviceArray.from_numpy(ids)
    d_sample = capi.DeviceArray((sample_num, dim), np.float32)
    d_centroids = capi.DeviceArray((c, dim), np.float32)
    wb = capi.kmeans_workspace_bytes(c, dim)
    ws = capi.DeviceArray(wb // 4 + 1, np.uint32)
    sb = capi.kmeans_seed_workspace_bytes(sample_num)
    seed_ws = capi.DeviceArray(sb // 8 + 1, np.uint64)
    with _Timer() as t:
        capi.sample_rows(d_data, dim, d_ids, sample_num, d_sample)
        capi.kmeans_seed(d_sample, sample_num, dim, c, param.seed, d_centroids, seed_ws, sb)
        capi.kmeans_fit(d_sample, sample_num, dim, c, param.kmeans_iterations, d_centroids, ws, wb)
    times["centroids"] = t.seconds
    # define_partition (partition.cuh:61-116)
    d_seg_idx = capi.DeviceArray((num, 3), np.uint32)
    d_seg_len = capi.DeviceArray(c + 1, np.uint32)
    wb = capi.partition_assign_workspace_bytes(num, c)
    ws = capi.DeviceArray(wb // 4 + 1, np.uint32)
    with _Timer() as t:
        capi.partition_assign(d_data, num, dim, d_centroids, c, param.boundary_factor, param.metric, d_seg_idx, d_seg_len,
                              None, ws, wb)
    times["assign"] = t.seconds
    h_len = d_seg_len.numpy()
    h_start = np.zeros(c + 1, dtype=np.uint32)
    h_start[1:] = np.cumsum(h_len[:-1], dtype=np.uint64).astype(np.uint32)
    reorder_num = num + int(h_len[c])
    # reorder (partition.cuh:118-157)
    d_reorder = capi.DeviceArray((reorder_num, dim), np.float32)
    d_map = capi.DeviceArray(reorder_num, np.uint32)
    d_start = capi.DeviceArray.from_numpy(h_start)
    with _Timer() as t:
        capi.reorder(d_data, num, dim, d_seg_idx, d_start, d_reorder, d_map)
    times["reorder"] = t.seconds
    if result is not None:
        result["pre_time"] = sum(times.values())
        result["pre_stages"] = times
    return d_reorder, d_map, h_start, h_len, d_centroids


def build_nnd(param, d_reorder_data, h_segment_start, h_segment_length, result=None, stats=False):
    """nn_descent.cuh:1405-1467.  Returns the kNN graph as a DeviceArray (reorder_num, graph_degree) of
    partition-local ids."""
    num, dim = d_reorder_data.shape
    degree = min(param.graph_degree, param.intermediate_graph_degree)
    d_ss = capi.DeviceArray.from_numpy(np.ascontiguousarray(h_segment_start, dtype=np.uint32))
    d_sl = capi.DeviceArray.from_numpy(np.ascontiguousarray(h_segment_length, dtype=np.uint32))
    d_knn = capi.DeviceArray((num, degree), np.uint32)
    wb = capi.nnd_workspace_bytes(num, dim, degree)
    ws = capi.DeviceArray(wb // 16 + 1, np.dtype("V16"))
    d_stats = capi.DeviceArray.from_numpy(np.zeros(2, np.uint64)) if stats else None
    with _Timer() as t:
        capi.nnd_build(d_reorder_data, num, dim, d_ss, d_sl, len(h_segment_start), degree, param.max_iterations,
                       param.termination_threshold, param.seed,
                       d_knn, ws, wb, d_stats)
    ws.free()
    if result is not None:
        result["knn_time"] = t.seconds
        if stats:
            result["nnd_stats"] = d_stats.numpy().tolist()
    return d_knn


class GLIDE:
    """glide.cuh:14-125 for Data_t = float, Index_t = uint32_t."""

    def __init__(self, graph_degree, data, centroids, metric):
        """data: numpy (num, dim) float32 or DeviceArray; centroids likewise (glide_impl.cuh:15-30).  Rows of a length
        that is no multiple of four are held padded (pad_rows); dim() is then the padded length."""
        _check_sizes(0, graph_degree)
        self.metric = metric
        self.d_data = pad_rows(data)
        self.d_centroids = pad_rows(centroids)
        if self.d_centroids.shape[1] != self.d_data.shape[1]:
            raise ValueError("centroids of %d values for points of %d" % (self.d_centroids.shape[1], self.d_data.shape[1]))
        self._graph_degree = int(graph_degree)
        self.d_graph = capi.DeviceArray((self.num(), self._graph_degree), np.uint32)
        self.d_start_points = None

    # accessors (glide.cuh:81-125)
    def dim(self): return self.d_data.shape[1]
    def num(self): return self.d_data.shape[0]
    def graph_degree(self): return self._graph_degree
    def centroid_num(self): return self.d_centroids.shape[0]
    def start_point_num(self): return self.d_start_points.shape[0]
    def data_view(self): return self.d_data
    def graph_view(self): return self.d_graph
    def centroid_view(self): return self.d_centroids
    def start_point_view(self): return self.d_start_points

    def load(self, h_graph, h_start_points):                                   # glide_impl.cuh:32-41
        self.d_graph.upload(np.ascontiguousarray(h_graph, dtype=np.uint32))
        self.d_start_points = capi.DeviceArray.from_numpy(np.ascontiguousarray(h_start_points, dtype=np.uint32))

    def start_point_select(self, h_segment_start, h_segment_length, h_map, seed):   # glide_impl.cuh:43-75
        rng = np.random.default_rng(seed)
        c = self.centroid_num()
        reorder_sp = np.zeros(len(h_segment_start), dtype=np.uint32)
        sp = np.zeros(c, dtype=np.uint32)
        for i in range(len(h_segment_start)):
            length = int(h_segment_length[i])
            reorder_sp[i] = rng.integers(0, length) if length > 0 else 0   # the reference underflows on an empty segment
            if i != c:
                sp[i] = h_map[int(h_segment_start[i]) + int(reorder_sp[i])] if length > 0 else 0
        return reorder_sp, sp

    def build(self, build_param, search_param_knn, search_param_refine, d_knn_graph, h_segment_start, h_segment_length,
              d_map, d_reorder_data, result=None, counters=False):
        """glide_impl.cuh:319-368: start points -> sub-graph build + boundary merge -> reverse edges -> refine.
        d_knn_graph, d_map and d_reorder_data are consumed (freed), as the reference resets its optionals."""
        num, dim, deg = self.num(), self.dim(), self._graph_degree
        knn_degree = d_knn_graph.shape[1]
        _check_sizes(search_param_knn.beam, knn_degree)
        _check_sizes(search_param_refine.beam, deg)
        reorder_num = d_reorder_data.shape[0]
        h_map = d_map.numpy()
        reorder_sp, sp = self.start_point_select(h_segment_start, h_segment_length, h_map, build_param.seed)
        d_ss = capi.DeviceArray.from_numpy(np.ascontiguousarray(h_segment_start, dtype=np.uint32))
        d_sl = capi.DeviceArray.from_numpy(np.ascontiguousarray(h_segment_length, dtype=np.uint32))
        d_rsp = capi.DeviceArray.from_numpy(reorder_sp)
        cnt = capi.new_counters() if counters else None
        times = {}
        p = search_param_knn
        with _Timer() as t:
            capi.build_subgraph(d_reorder_data, num, dim, d_knn_graph, knn_degree, d_map, d_ss, d_sl, len(h_segment_start), d_rsp,
                                deg, p.beam, p.max_iterations, p.min_iterations, p.hash_bit, p.hash_reset_interval,
                                build_param.relaxant_factor, self.metric, self.d_graph, cnt)
        times["subgraph"] = t.seconds
        with _Timer() as t:
            if reorder_num > num:
                capi.build_boundary(d_reorder_data, num, reorder_num, dim, d_knn_graph, knn_degree, d_map,
                                    int(reorder_sp[self.centroid_num()]), deg, p.beam, p.max_iterations, p.min_iterations,
                                    p.hash_bit, p.hash_reset_interval, build_param.relaxant_factor, self.metric, self.d_graph, cnt)
        times["boundary"] = t.seconds
        if counters and result is not None:
            capi.synchronize()
            result["build_counters"] = capi.read_counters(cnt)
        for consumed in (d_knn_graph, d_reorder_data):     # d_map is kept until the refine stage, which uses it as its order
            capi.synchronize()
            consumed.free()
        self.d_start_points = capi.DeviceArray.from_numpy(sp)
        # reverse_graph (glide_impl.cuh:194-256)
        d_rev = capi.DeviceArray((num, deg), np.uint32)
        d_rcnt = capi.DeviceArray(num, np.uint32)
        wb = capi.reverse_edges_workspace_bytes(num, deg)
        ws = capi.DeviceArray(wb // 8 + 1, np.uint64)
        with _Timer() as t:
            capi.reverse_edges(self.d_graph, num, deg, d_rev, d_rcnt, ws, wb)
            capi.insert_reverse(self.d_graph, d_rev, d_rcnt, num, deg)
        times["reverse"] = t.seconds
        ws.free()
        d_rcnt.free()
        # refine (glide_impl.cuh:258-316); d_rev is reused as the output graph
        times["refine"] = 0.0
        if search_param_refine.beam != 0:
            p = search_param_refine
            cnt2 = capi.new_counters() if counters else None
            with _Timer() as t:
                capi.refine(self.d_data, num, dim, self.d_graph, d_rev, deg, self.d_centroids, self.centroid_num(),
                            self.d_start_points, p.beam, p.max_iterations, p.min_iterations, p.hash_bit, p.hash_reset_interval,
                            build_param.relaxant_factor, self.metric, cnt2, order=d_map)
            times["refine"] = t.seconds
            self.d_graph, d_rev = d_rev, self.d_graph
            if counters and result is not None:
                result["refine_counters"] = capi.read_counters(cnt2)
        d_rev.free()
        d_map.free()
        if result is not None:
            result["index_time"] = times["subgraph"] + times["boundary"] + times["reverse"]
            result["refine_time"] = times["refine"]
            result["build_stages"] = times

    def search(self, param, d_query, result=None, counters=None, stream=None, out=None):
        """glide_impl.cuh:370-454.  d_query: DeviceArray (query_num, dim), in the data's own row length or padded as
        the data is held.  Returns (ids, dists) as numpy arrays unless `out` = (d_ids, d_dists) is given, in which case
        nothing is copied back."""
        _check_sizes(param.beam, self._graph_degree)
        d_query = pad_rows(d_query)
        if d_query.shape[1] != self.dim():
            raise ValueError("queries of %d values for points of %d" % (d_query.shape[1], self.dim()))
        nq = d_query.shape[0]
        d_ids, d_dists = out if out is not None else (capi.DeviceArray((nq, param.top_k), np.uint32), capi.DeviceArray((nq, param.top_k), np.float32))
        with _Timer() as t:
            capi.search(self.d_data, self.num(), self.dim(), self.d_graph, self._graph_degree, self.d_centroids, self.centroid_num(),
                        self.d_start_points, d_query, nq, param.top_k, param.beam, param.max_iterations, param.min_iterations,
                        param.hash_bit, param.hash_reset_interval, self.metric, d_ids, d_dists, counters, stream)
        if result is not None:
            result["search_time"] = t.seconds
            result["QPS"] = nq / t.seconds if t.seconds > 0 else float("inf")
        if out is not None:
            return None
        return d_ids.numpy(), d_dists.numpy()
