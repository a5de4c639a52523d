"""ctypes binding of libglide_hip.so (the C ABI declared in include/glide_hip.h).

The library is the product; this module only marshals arguments.  There is no CPU fallback: if the shared
library is missing or a call fails, an exception is raised.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("GLIDE_HIP_LIB", os.path.join(_HERE, "libglide_hip.so"))   # override: an alternative build of the library
_lib = None

EUCLIDEAN, COSINE = 0, 1
INVALID = 0xFFFFFFFF

u32, f32, vp = C.c_uint32, C.c_float, C.c_void_p


class GlideHipError(RuntimeError):
    def __init__(self, code, what):
        self.code = code
        super().__init__("%s failed: %s (code %d)" % (what, error_string(code), code))


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libglide_hip.so is not built: run `python -c 'import __graft_entry__ as g; g.build()'` "
                               "or `make -C glide_amd/csrc`")
        _lib = C.CDLL(LIB_PATH)
        _lib.glide_hip_version.restype = C.c_char_p
        _lib.glide_hip_error_string.restype = C.c_char_p
    return _lib


def error_string(code):
    return lib().glide_hip_error_string(C.c_int(code)).decode()


def check(code, what):
    if code != 0:
        raise GlideHipError(code, what)


def version():
    return lib().glide_hip_version().decode()


def set_device(device=0):
    check(lib().glide_hip_set_device(C.c_int(device)), "glide_hip_set_device")


def device_info():
    name = C.create_string_buffer(256)
    cus, mem = C.c_int(0), C.c_size_t(0)
    check(lib().glide_hip_device_info(name, C.c_size_t(256), C.byref(cus), C.byref(mem)), "glide_hip_device_info")
    return dict(name=name.value.decode(), compute_units=cus.value, total_mem=mem.value)


class DeviceArray:
    """A typed device allocation owned through glide_hip_malloc / glide_hip_free."""

    def __init__(self, shape, dtype):
        self.shape = tuple(int(s) for s in (shape if isinstance(shape, (tuple, list)) else (shape,)))
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        p = vp()
        check(lib().glide_hip_malloc(C.byref(p), C.c_size_t(self.nbytes)), "glide_hip_malloc")
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, arr, dtype=None):
        arr = np.ascontiguousarray(arr, dtype=dtype)
        d = cls(arr.shape, arr.dtype)
        d.upload(arr)
        return d

    @classmethod
    def full(cls, shape, value, dtype=np.uint32):
        d = cls(shape, dtype)
        assert d.dtype.itemsize == 4
        v = int(np.array([value], dtype=d.dtype).view(np.uint32)[0])
        check(lib().glide_hip_fill_u32(vp(d.ptr), u32(v), C.c_size_t(d.nbytes // 4), None), "glide_hip_fill_u32")
        return d

    def upload(self, arr):
        arr = np.ascontiguousarray(arr, dtype=self.dtype)
        assert arr.nbytes == self.nbytes
        check(lib().glide_hip_memcpy_h2d(vp(self.ptr), arr.ctypes.data_as(vp), C.c_size_t(self.nbytes), None),
              "glide_hip_memcpy_h2d")

    def numpy(self):
        out = np.empty(self.shape, dtype=self.dtype)
        check(lib().glide_hip_memcpy_d2h(out.ctypes.data_as(vp), vp(self.ptr), C.c_size_t(self.nbytes), None),
              "glide_hip_memcpy_d2h")
        return out

    def free(self):
        if self.ptr:
            lib().glide_hip_free(vp(self.ptr))
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


COUNTER_STRIPES = 256


def new_counters():
    """Zeroed device counters for the beam kernels (COUNTER_STRIPES x 3 u64)."""
    return DeviceArray.from_numpy(np.zeros((COUNTER_STRIPES, 3), np.uint64))


def read_counters(counters):
    """[beam iterations, data rows scored, graph rows read] summed over the stripes."""
    return counters.numpy().sum(0).tolist()


def _ptr(x):
    """Device pointer of a DeviceArray, a torch tensor, a raw int, or None."""
    if x is None:
        return vp(None)
    if isinstance(x, DeviceArray):
        return vp(x.ptr)
    if isinstance(x, int):
        return vp(x)
    if hasattr(x, "data_ptr"):
        return vp(x.data_ptr())
    raise TypeError("not a device buffer: %r" % type(x))


def synchronize(stream=None):
    check(lib().glide_hip_stream_synchronize(vp(stream)), "glide_hip_stream_synchronize")


class Event:
    def __init__(self):
        p = vp()
        check(lib().glide_hip_event_create(C.byref(p)), "glide_hip_event_create")
        self.ptr = p.value

    def record(self, stream=None):
        check(lib().glide_hip_event_record(vp(self.ptr), vp(stream)), "glide_hip_event_record")

    def elapsed_ms(self, stop):
        ms = f32(0)
        check(lib().glide_hip_event_elapsed_ms(vp(self.ptr), vp(stop.ptr), C.byref(ms)), "glide_hip_event_elapsed_ms")
        return ms.value

    def __del__(self):
        try:
            if self.ptr:
                lib().glide_hip_event_destroy(vp(self.ptr))
        except Exception:
            pass


# ------------------------------------------------------------------------------------------- entry points
def search(data, num, dim, graph, graph_degree, centroids, centroid_num, start_points, queries, query_num, top_k,
           beam, max_iterations, min_iterations, hash_bit, hash_reset_interval, metric, result_ids, result_dists,
           counters=None, stream=None):
    check(lib().glide_hip_search(_ptr(data), u32(num), u32(dim), _ptr(graph), u32(graph_degree), _ptr(centroids),
                                 u32(centroid_num), _ptr(start_points), _ptr(queries), u32(query_num), u32(top_k),
                                 u32(beam), u32(max_iterations), u32(min_iterations), u32(hash_bit),
                                 u32(hash_reset_interval), C.c_int(metric), _ptr(result_ids), _ptr(result_dists),
                                 _ptr(counters), vp(stream)), "glide_hip_search")


def search_merged(data, num, dim, graph, graph_degree, centroids, centroid_num, start_points, queries, query_num, top_k,
                  beam, max_iterations, min_iterations, hash_bit, hash_reset_interval, metric, result_ids, result_dists,
                  counters=None, stream=None):
    check(lib().glide_hip_search_merged(_ptr(data), u32(num), u32(dim), _ptr(graph), u32(graph_degree), _ptr(centroids),
                                        u32(centroid_num), _ptr(start_points), _ptr(queries), u32(query_num), u32(top_k),
                                        u32(beam), u32(max_iterations), u32(min_iterations), u32(hash_bit),
                                        u32(hash_reset_interval), C.c_int(metric), _ptr(result_ids), _ptr(result_dists),
                                        _ptr(counters), vp(stream)), "glide_hip_search_merged")


def distance_batch(a, b, n, dim, metric, out, stream=None):
    check(lib().glide_hip_distance_batch(_ptr(a), _ptr(b), u32(n), u32(dim), C.c_int(metric), _ptr(out), vp(stream)),
          "glide_hip_distance_batch")


def bitonic_sort_kv(keys, vals, m, batch, stream=None):
    check(lib().glide_hip_bitonic_sort_kv(_ptr(keys), _ptr(vals), u32(m), u32(batch), vp(stream)),
          "glide_hip_bitonic_sort_kv")


def bitonic_merge_kv(keys, vals, m, batch, stream=None):
    check(lib().glide_hip_bitonic_merge_kv(_ptr(keys), _ptr(vals), u32(m), u32(batch), vp(stream)),
          "glide_hip_bitonic_merge_kv")


def hashmap_insert_seq(table, bitlen, keys, n, flags, stream=None):
    check(lib().glide_hip_hashmap_insert_seq(_ptr(table), u32(bitlen), _ptr(keys), u32(n), _ptr(flags), vp(stream)),
          "glide_hip_hashmap_insert_seq")


def build_subgraph(reorder_data, num, dim, knn_graph, knn_degree, mp, segment_starts, segment_lengths, segment_num,
                   start_points, graph_degree, beam, max_iterations, min_iterations, hash_bit, hash_reset_interval,
                   relaxant, metric, graph, counters=None, stream=None):
    check(lib().glide_hip_build_subgraph(_ptr(reorder_data), u32(num), u32(dim), _ptr(knn_graph), u32(knn_degree),
                                         _ptr(mp), _ptr(segment_starts), _ptr(segment_lengths), u32(segment_num),
                                         _ptr(start_points), u32(graph_degree), u32(beam), u32(max_iterations),
                                         u32(min_iterations), u32(hash_bit), u32(hash_reset_interval), f32(relaxant),
                                         C.c_int(metric), _ptr(graph), _ptr(counters), vp(stream)),
          "glide_hip_build_subgraph")


def build_boundary(reorder_data, num, reorder_num, dim, knn_graph, knn_degree, mp, start_point, graph_degree, beam,
                   max_iterations, min_iterations, hash_bit, hash_reset_interval, relaxant, metric, graph,
                   counters=None, stream=None):
    check(lib().glide_hip_build_boundary(_ptr(reorder_data), u32(num), u32(reorder_num), u32(dim), _ptr(knn_graph),
                                         u32(knn_degree), _ptr(mp), u32(start_point), u32(graph_degree), u32(beam),
                                         u32(max_iterations), u32(min_iterations), u32(hash_bit),
                                         u32(hash_reset_interval), f32(relaxant), C.c_int(metric), _ptr(graph),
                                         _ptr(counters), vp(stream)), "glide_hip_build_boundary")


def reverse_edges_workspace_bytes(num, graph_degree):
    f = lib().glide_hip_reverse_edges_workspace_bytes
    f.restype = C.c_size_t
    return int(f(u32(num), u32(graph_degree)))


def reverse_edges(graph, num, graph_degree, reverse_graph, reverse_counts, workspace, workspace_bytes, stream=None):
    check(lib().glide_hip_reverse_edges(_ptr(graph), u32(num), u32(graph_degree), _ptr(reverse_graph),
                                        _ptr(reverse_counts), _ptr(workspace), C.c_size_t(workspace_bytes),
                                        vp(stream)), "glide_hip_reverse_edges")


def insert_reverse(graph, reverse_graph, reverse_counts, num, graph_degree, stream=None):
    check(lib().glide_hip_insert_reverse(_ptr(graph), _ptr(reverse_graph), _ptr(reverse_counts), u32(num),
                                         u32(graph_degree), vp(stream)), "glide_hip_insert_reverse")


def refine(data, num, dim, graph_in, graph_out, graph_degree, centroids, centroid_num, start_points, beam,
           max_iterations, min_iterations, hash_bit, hash_reset_interval, relaxant, metric, counters=None,
           stream=None, order=None):
    check(lib().glide_hip_refine(_ptr(data), u32(num), u32(dim), _ptr(graph_in), _ptr(graph_out), u32(graph_degree),
                                 _ptr(centroids), u32(centroid_num), _ptr(start_points), u32(beam),
                                 u32(max_iterations), u32(min_iterations), u32(hash_bit), u32(hash_reset_interval),
                                 f32(relaxant), C.c_int(metric), _ptr(order), _ptr(counters), vp(stream)), "glide_hip_refine")


def refine_merged(data, num, dim, graph_in, graph_out, graph_degree, centroids, centroid_num, start_points, beam,
           max_iterations, min_iterations, hash_bit, hash_reset_interval, relaxant, metric, counters=None,
           stream=None, order=None):
    check(lib().glide_hip_refine_merged(_ptr(data), u32(num), u32(dim), _ptr(graph_in), _ptr(graph_out), u32(graph_degree),
                                 _ptr(centroids), u32(centroid_num), _ptr(start_points), u32(beam),
                                 u32(max_iterations), u32(min_iterations), u32(hash_bit), u32(hash_reset_interval),
                                 f32(relaxant), C.c_int(metric), _ptr(order), _ptr(counters), vp(stream)), "glide_hip_refine_merged")


def _size_fn(name):
    f = getattr(lib(), name)
    f.restype = C.c_size_t
    return f


def partition_assign_workspace_bytes(num, centroid_num):
    return int(_size_fn("glide_hip_partition_assign_workspace_bytes")(u32(num), u32(centroid_num)))


def partition_assign(data, num, dim, centroids, centroid_num, boundary_factor, metric, segment_indexes,
                     segment_lengths, nearest_dists, workspace, workspace_bytes, stream=None):
    check(lib().glide_hip_partition_assign(_ptr(data), u32(num), u32(dim), _ptr(centroids), u32(centroid_num),
                                           f32(boundary_factor), C.c_int(metric), _ptr(segment_indexes),
                                           _ptr(segment_lengths), _ptr(nearest_dists), _ptr(workspace),
                                           C.c_size_t(workspace_bytes), vp(stream)), "glide_hip_partition_assign")


def mem_info():
    """(free, total) bytes of device memory on the current device."""
    free, total = C.c_size_t(0), C.c_size_t(0)
    check(lib().glide_hip_mem_info(C.byref(free), C.byref(total)), "glide_hip_mem_info")
    return free.value, total.value


def partition_assign_fixed_max_points():
    f = lib().glide_hip_partition_assign_fixed_max_points
    f.restype = C.c_uint32
    return int(f())


def partition_assign_fixed(data, num, dim, centroids, centroid_num, boundary_factor, metric, segment_indexes,
                           segment_lengths, nearest_dists, stream=None, check_status=True):
    rc = lib().glide_hip_partition_assign_fixed(_ptr(data), u32(num), u32(dim), _ptr(centroids), u32(centroid_num),
                                                f32(boundary_factor), C.c_int(metric), _ptr(segment_indexes),
                                                _ptr(segment_lengths), _ptr(nearest_dists), vp(stream))
    if check_status:
        check(rc, "glide_hip_partition_assign_fixed")
    return rc


def reorder(data, num, dim, segment_indexes, segment_starts, reorder_data, mp, stream=None):
    check(lib().glide_hip_reorder(_ptr(data), u32(num), u32(dim), _ptr(segment_indexes), _ptr(segment_starts),
                                  _ptr(reorder_data), _ptr(mp), vp(stream)), "glide_hip_reorder")


def sample_rows(data, dim, sample_ids, sample_num, sample, stream=None):
    check(lib().glide_hip_sample_rows(_ptr(data), u32(dim), _ptr(sample_ids), u32(sample_num), _ptr(sample),
                                      vp(stream)), "glide_hip_sample_rows")


def kmeans_workspace_bytes(cluster_num, dim):
    return int(_size_fn("glide_hip_kmeans_workspace_bytes")(u32(cluster_num), u32(dim)))


def kmeans_seed_workspace_bytes(sample_num):
    return int(_size_fn("glide_hip_kmeans_seed_workspace_bytes")(u32(sample_num)))


def kmeans_seed(sample, sample_num, dim, cluster_num, seed, centroids, workspace, workspace_bytes, chosen_rows=None, stream=None):
    check(lib().glide_hip_kmeans_seed(_ptr(sample), u32(sample_num), u32(dim), u32(cluster_num), u32(seed), _ptr(centroids),
                                      _ptr(chosen_rows), _ptr(workspace), C.c_size_t(workspace_bytes), vp(stream)), "glide_hip_kmeans_seed")


def kmeans_fit(sample, sample_num, dim, cluster_num, iterations, centroids, workspace, workspace_bytes, stream=None):
    check(lib().glide_hip_kmeans_fit(_ptr(sample), u32(sample_num), u32(dim), u32(cluster_num), u32(iterations),
                                     _ptr(centroids), _ptr(workspace), C.c_size_t(workspace_bytes), vp(stream)),
          "glide_hip_kmeans_fit")


def nnd_workspace_bytes(reorder_num, dim, knn_degree):
    return int(_size_fn("glide_hip_nnd_workspace_bytes")(u32(reorder_num), u32(dim), u32(knn_degree)))


def nnd_build(reorder_data, reorder_num, dim, segment_starts, segment_lengths, segment_num, knn_degree, iterations,
              termination_threshold, seed, knn_graph, workspace, workspace_bytes, stats=None, stream=None):
    check(lib().glide_hip_nnd_build(_ptr(reorder_data), u32(reorder_num), u32(dim), _ptr(segment_starts),
                                    _ptr(segment_lengths), u32(segment_num), u32(knn_degree), u32(iterations),
                                    f32(termination_threshold), u32(seed), _ptr(knn_graph), _ptr(workspace),
                                    C.c_size_t(workspace_bytes), _ptr(stats), vp(stream)), "glide_hip_nnd_build")


class NndLayout(C.Structure):
    """glide_nnd_layout: byte offsets of the NN-descent arrays inside the workspace."""
    _fields_ = [(n, C.c_uint64) for n in ("half_rows", "norms", "list_ids", "list_dists", "fwd_new", "fwd_old", "rev_new", "rev_old",
                                          "rev_tables", "rev_thr", "counts", "members", "member_counts", "offers", "bloom", "segment_state", "segment_updates", "round", "total")] + \
               [(n, C.c_uint32) for n in ("width", "reverse_cap", "reverse_stride", "offer_slots", "reverse_slots", "row_halfs", "bloom_sets", "reserved")]


def nnd_layout(reorder_num, dim, knn_degree):
    out = NndLayout()
    check(lib().glide_hip_nnd_layout(u32(reorder_num), u32(dim), u32(knn_degree), C.byref(out)), "glide_hip_nnd_layout")
    return out


def _nnd_stage(name, reorder_num, dim, segment_starts, segment_lengths, segment_num, knn_degree, workspace, workspace_bytes, stream):
    check(getattr(lib(), name)(u32(reorder_num), u32(dim), _ptr(segment_starts), _ptr(segment_lengths), u32(segment_num),
                               u32(knn_degree), _ptr(workspace), C.c_size_t(workspace_bytes), vp(stream)), name)


def nnd_prepare(reorder_data, reorder_num, dim, segment_starts, segment_lengths, segment_num, knn_degree, seed, workspace,
                workspace_bytes, stream=None):
    check(lib().glide_hip_nnd_prepare(_ptr(reorder_data), u32(reorder_num), u32(dim), _ptr(segment_starts), _ptr(segment_lengths),
                                      u32(segment_num), u32(knn_degree), u32(seed), _ptr(workspace), C.c_size_t(workspace_bytes),
                                      vp(stream)), "glide_hip_nnd_prepare")


def nnd_sample(*args, stream=None):
    _nnd_stage("glide_hip_nnd_sample", *args, stream)


def nnd_reverse_sample(*args, stream=None):
    _nnd_stage("glide_hip_nnd_reverse_sample", *args, stream)


def nnd_local_join(*args, stream=None):
    _nnd_stage("glide_hip_nnd_local_join", *args, stream)


def nnd_merge(*args, stream=None):
    _nnd_stage("glide_hip_nnd_merge", *args, stream)


def nnd_converge(reorder_num, dim, segment_starts, segment_lengths, segment_num, knn_degree, termination_threshold, workspace,
                 workspace_bytes, stream=None):
    check(lib().glide_hip_nnd_converge(u32(reorder_num), u32(dim), _ptr(segment_starts), _ptr(segment_lengths), u32(segment_num),
                                       u32(knn_degree), f32(termination_threshold), _ptr(workspace), C.c_size_t(workspace_bytes),
                                       vp(stream)), "glide_hip_nnd_converge")


def nnd_finalize(reorder_num, dim, segment_starts, segment_lengths, segment_num, knn_degree, knn_graph, stats, workspace,
                 workspace_bytes, stream=None):
    check(lib().glide_hip_nnd_finalize(u32(reorder_num), u32(dim), _ptr(segment_starts), _ptr(segment_lengths), u32(segment_num),
                                       u32(knn_degree), _ptr(knn_graph), _ptr(stats), _ptr(workspace), C.c_size_t(workspace_bytes),
                                       vp(stream)), "glide_hip_nnd_finalize")


def widen_u8(src, count, dst, stream=None):
    check(lib().glide_hip_widen_u8(_ptr(src), C.c_size_t(count), _ptr(dst), vp(stream)), "glide_hip_widen_u8")


def copy_rows(src, num, src_dim, dst, dst_dim, stream=None):
    check(lib().glide_hip_copy_rows(_ptr(src), C.c_uint64(num), C.c_uint32(src_dim), _ptr(dst), C.c_uint32(dst_dim), vp(stream)),
          "glide_hip_copy_rows")


def build_segment(segment_data, num, dim, knn_graph, knn_degree, start_point, graph_degree, beam, max_iterations,
                  min_iterations, hash_bit, hash_reset_interval, relaxant, metric, graph, counters=None, stream=None):
    check(lib().glide_hip_build_segment(_ptr(segment_data), u32(num), u32(dim), _ptr(knn_graph), u32(knn_degree),
                                        u32(start_point), u32(graph_degree), u32(beam), u32(max_iterations),
                                        u32(min_iterations), u32(hash_bit), u32(hash_reset_interval), f32(relaxant),
                                        C.c_int(metric), _ptr(graph), _ptr(counters), vp(stream)), "glide_hip_build_segment")


def place_segment_graph(segment_graph, segment_length, graph_degree, segment_start, merged_graph, stream=None):
    check(lib().glide_hip_place_segment_graph(_ptr(segment_graph), u32(segment_length), u32(graph_degree), u32(segment_start),
                                              _ptr(merged_graph), vp(stream)), "glide_hip_place_segment_graph")


def merge_boundary_graph(boundary_graph, boundary_num, graph_degree, home_rows, merged_graph, stream=None):
    check(lib().glide_hip_merge_boundary_graph(_ptr(boundary_graph), u32(boundary_num), u32(graph_degree), _ptr(home_rows),
                                               _ptr(merged_graph), vp(stream)), "glide_hip_merge_boundary_graph")


def refine_segment(segment_data, num, dim, graph_in, graph_out, graph_degree, start_point, beam, max_iterations,
                   min_iterations, hash_bit, hash_reset_interval, relaxant, metric, counters=None, stream=None):
    check(lib().glide_hip_refine_segment(_ptr(segment_data), u32(num), u32(dim), _ptr(graph_in), _ptr(graph_out),
                                         u32(graph_degree), u32(start_point), u32(beam), u32(max_iterations),
                                         u32(min_iterations), u32(hash_bit), u32(hash_reset_interval), f32(relaxant),
                                         C.c_int(metric), _ptr(counters), vp(stream)), "glide_hip_refine_segment")


def select_segments(queries, query_num, dim, centroids, centroid_num, min_segment_num, boundary_factor, metric,
                    segment_ids, stream=None):
    check(lib().glide_hip_select_segments(_ptr(queries), u32(query_num), u32(dim), _ptr(centroids), u32(centroid_num),
                                          u32(min_segment_num), f32(boundary_factor), C.c_int(metric),
                                          _ptr(segment_ids), vp(stream)), "glide_hip_select_segments")


def group_queries(segment_ids, query_num, centroid_num, counts, offsets, lists, stream=None):
    wb = int(_size_fn("glide_hip_group_queries_workspace_bytes")(u32(centroid_num)))
    ws = DeviceArray(wb // 4 + 1, np.uint32)
    check(lib().glide_hip_group_queries(_ptr(segment_ids), u32(query_num), u32(centroid_num), _ptr(counts), _ptr(offsets), _ptr(lists),
                                        _ptr(ws), C.c_size_t(wb), vp(stream)), "glide_hip_group_queries")
    synchronize(stream)      # the workspace is released on return


def search_sub_listed(segment_data, dim, segment_graph, graph_degree, segment_map, queries, query_num, query_list, list_len,
                      segment_id, start_point, top_k, beam, max_iterations, min_iterations, hash_bit, hash_reset_interval, metric,
                      final_ids, final_dists, counters=None, stream=None):
    check(lib().glide_hip_search_sub_listed(_ptr(segment_data), u32(dim), _ptr(segment_graph), u32(graph_degree), _ptr(segment_map),
                                            _ptr(queries), u32(query_num), _ptr(query_list), u32(list_len), u32(segment_id),
                                            u32(start_point), u32(top_k), u32(beam), u32(max_iterations), u32(min_iterations),
                                            u32(hash_bit), u32(hash_reset_interval), C.c_int(metric), _ptr(final_ids), _ptr(final_dists),
                                            _ptr(counters), vp(stream)), "glide_hip_search_sub_listed")


def search_partitions(data, dim, graph, graph_degree, mp, segment_starts, segment_start_points, segment_num, queries, query_num,
                      segment_ids, top_k, beam, max_iterations, min_iterations, hash_bit, hash_reset_interval, metric, final_ids,
                      final_dists, counters=None, stream=None):
    wb = int(_size_fn("glide_hip_search_partitions_workspace_bytes")(u32(query_num), u32(segment_num), u32(top_k)))
    ws = DeviceArray(wb // 8 + 1, np.uint64)
    check(lib().glide_hip_search_partitions(_ptr(data), u32(dim), _ptr(graph), u32(graph_degree), _ptr(mp), _ptr(segment_starts),
                                            _ptr(segment_start_points), u32(segment_num), _ptr(queries), u32(query_num), _ptr(segment_ids),
                                            u32(top_k), u32(beam), u32(max_iterations), u32(min_iterations), u32(hash_bit),
                                            u32(hash_reset_interval), C.c_int(metric), _ptr(final_ids), _ptr(final_dists), _ptr(ws),
                                            C.c_size_t(wb), _ptr(counters), vp(stream)), "glide_hip_search_partitions")
    synchronize(stream)      # the workspace is released on return


def search_sub(segment_data, dim, segment_graph, graph_degree, segment_map, queries, query_num, segment_ids,
               centroid_num, segment_id, start_point, top_k, beam, max_iterations, min_iterations, hash_bit,
               hash_reset_interval, metric, final_ids, final_dists, counters=None, stream=None):
    check(lib().glide_hip_search_sub(_ptr(segment_data), u32(dim), _ptr(segment_graph), u32(graph_degree),
                                     _ptr(segment_map), _ptr(queries), u32(query_num), _ptr(segment_ids),
                                     u32(centroid_num), u32(segment_id), u32(start_point), u32(top_k), u32(beam),
                                     u32(max_iterations), u32(min_iterations), u32(hash_bit), u32(hash_reset_interval),
                                     C.c_int(metric), _ptr(final_ids), _ptr(final_dists), _ptr(counters), vp(stream)),
          "glide_hip_search_sub")
