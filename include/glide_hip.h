/*
 * glide_hip.h -- C ABI of the MI355X (gfx950) GLIDE kernels.
 *
 * Every entry point takes raw device pointers and plain sizes, launches on `stream` (a hipStream_t passed as
 * void*, NULL = default stream) and returns an int: 0 = success, > 0 = a hipError_t value, < 0 = one of the
 * GLIDE_ERR_* argument errors below.  No exceptions cross the boundary and the library keeps no global state.
 * Each declaration cites the interface of the reference implementation (owlet-hub/GLIDE, paths relative to its
 * src/ directory) that it replaces.
 *
 * Unless stated otherwise the kernels allocate nothing; entry points that need scratch memory say so and
 * allocate/free it with hipMallocAsync/hipFreeAsync on `stream`.
 */
#ifndef GLIDE_HIP_H
#define GLIDE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GLIDE_OK 0
#define GLIDE_ERR_UNSUPPORTED (-1) /* size outside the supported buckets (reference: std::invalid_argument, kernel_config.cuh:48,60) */
#define GLIDE_ERR_BAD_ARGUMENT (-2) /* null pointer, zero size, misaligned row */
#define GLIDE_ERR_NO_DEVICE (-3)

#define GLIDE_METRIC_EUCLIDEAN 0 /* params.cuh:5-8 */
#define GLIDE_METRIC_COSINE 1

#define GLIDE_INVALID_ID 0xffffffffu

/* ---- library / device ------------------------------------------------------------------------------------ */
const char *glide_hip_version(void);
const char *glide_hip_error_string(int code);
/* replaces the hard-coded cudaSetDevice(1) of the reference mains (small_build.cu:33) */
int glide_hip_set_device(int device);
int glide_hip_device_info(char *name, size_t name_len, int *compute_units, size_t *total_mem);

/* memory / stream / event helpers for hosts that have no HIP runtime of their own
 * (replace raft::make_device_matrix / raft::copy / rmm stream pool / cudaEvent use, glide_impl.cuh:15-41,53-72) */
int glide_hip_malloc(void **ptr, size_t bytes);
int glide_hip_free(void *ptr);
int glide_hip_host_alloc_pinned(void **ptr, size_t bytes);
int glide_hip_host_free_pinned(void *ptr);
int glide_hip_memcpy_h2d(void *dst, const void *src, size_t bytes, void *stream);
int glide_hip_memcpy_d2h(void *dst, const void *src, size_t bytes, void *stream);
int glide_hip_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream);
int glide_hip_fill_u32(uint32_t *ptr, uint32_t value, size_t count, void *stream); /* thrust::fill sites */
int glide_hip_stream_create(void **stream);
int glide_hip_stream_destroy(void *stream);
int glide_hip_stream_synchronize(void *stream);
int glide_hip_event_create(void **event);
int glide_hip_event_destroy(void *event);
int glide_hip_event_record(void *event, void *stream);
int glide_hip_event_elapsed_ms(void *start, void *stop, float *ms); /* synchronises on `stop` */

/* ---- beam search (subsystem 4) ----------------------------------------------------------------------------
 * Replaces search_kernel<MAX_CANDIDATE,MAX_BEAM,MAX_CENTROID> (search_kernel.cuh:393-490) as launched by
 * GLIDE::search (glide_impl.cuh:370-454).  One query per wavefront.  result_ids/result_dists are
 * query_num x top_k.  `counters` (nullable) receives three u64 sums: beam iterations, data rows scored, graph
 * rows read -- the algorithmic-traffic tallies.
 * Limits: graph_degree <= 128, beam <= 256, centroid_num <= 256, dim % 4 == 0, dim <= 1024, top_k <= beam. */
int glide_hip_search(const float *data, uint32_t num, uint32_t dim, const uint32_t *graph, uint32_t graph_degree,
                     const float *centroids, uint32_t centroid_num, const uint32_t *start_points,
                     const float *queries, uint32_t query_num, uint32_t top_k, uint32_t beam,
                     uint32_t max_iterations, uint32_t min_iterations, uint32_t hash_bit,
                     uint32_t hash_reset_interval, int metric, uint32_t *result_ids, float *result_dists,
                     unsigned long long *counters, void *stream);

/* ---- test hooks for the device primitives (subsystems 5, 6 and the hash set) ------------------------------ */
/* compute_similarity_warp (distance.cuh:9-27): out[i] = dist(a[i], b[i]) for n row pairs */
int glide_hip_distance_batch(const float *a, const float *b, uint32_t n, uint32_t dim, int metric, float *out,
                             void *stream);
/* bitonic::warp_sort (bitonic.cuh:207-212): each of `batch` arrays of m (32..512, power of two) pairs is
 * sorted by one wavefront; arrays are in network element order */
int glide_hip_bitonic_sort_kv(float *keys, uint32_t *vals, uint32_t m, uint32_t batch, void *stream);
/* bitonic::warp_merge with range 32 (bitonic.cuh:202-205) */
int glide_hip_bitonic_merge_kv(float *keys, uint32_t *vals, uint32_t m, uint32_t batch, void *stream);
/* hashmap::insert (hashmap.cuh:34-55), keys inserted one after another; table has 1 << bitlen words and must
 * be pre-filled with 0xffffffff (or carry earlier state); flags[i] = 1 iff keys[i] was newly stored */
int glide_hip_hashmap_insert_seq(uint32_t *table, uint32_t bitlen, const uint32_t *keys, uint32_t n,
                                 uint32_t *flags, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* GLIDE_HIP_H */
