/*
 * CPU oracle for the GLIDE build/search path.  TEST INFRASTRUCTURE ONLY.
 *
 * This is a sequential/OpenMP restatement of the reference's algorithms, used as the checker
 * for the HIP kernels and as the timed CPU baseline.  Nothing in the product path (the HIP
 * library, the C++ host layer, the Python wrapper) may link, import or call it.
 *
 * Every function cites the reference file:line it follows (paths relative to the reference's src/).
 *
 * Pinning status (what fixes each function's output independently of this restatement):
 *   params                 hand-computed table + closed forms                       (pinned)
 *   bitonic sort / merge   distinct keys == std::sort, 0/1 principle on small M,
 *                          tie behaviour = literal comparator sequence of bitonic.cuh (pinned)
 *   two-warp sort / merge  (degree > 128, beam > 256) distinct keys: the smallest `beam` keys in
 *                          ascending order == std::sort (pinned); ties follow the reference's
 *                          comparator and shared-memory sequence as written
 *   hashmap                hand-derived table layouts, set invariants               (pinned)
 *   distance               float64 closed form, rel <= 1e-5                         (pinned)
 *   partition assign       float64 brute-force argmin / ratio test                  (pinned)
 *   prune                  RNG invariant over kept pairs, brute force on tiny pools (pinned)
 *   boundary merge         hand-worked rows for both branches                       (pinned)
 *   reverse edges          invariants + brute force                                 (pinned)
 *   beam search            recall vs exact brute force; the visited-set reset + restore by a hand-derived run
 *                          on a path graph (results, iterations, rows scored for six reset intervals, a table
 *                          that overflows unless it is cleared) and by equality with a reset-free search (pinned)
 *   refine                 hand-worked rows on a 12-point line graph + a float64 model written from the
 *                          definition (first admissible head, heads before it dropped, holes in slot order),
 *                          every row of random graphs with holes                    (pinned)
 *   segment choice         numpy: float64 distances, stable argsort, ratio test, top-up (pinned)
 *   large-path result merge  sorted union of the partitions' own top-k (from the small path's search),
 *                          any partition order, unlisted partitions and list gaps     (pinned)
 *   NN-descent             parity unpinned bit-wise (the reference is unseeded and racy);
 *                          statistical: graph recall vs exact kNN
 *   k-means (cuVS)         parity unpinned (third-party, absent from the reference tree); the stand-in
 *                          (greedy k-means++ seeding + Lloyd) is held to scikit-learn's inertia through
 *                          the fixture tests/golden/kmeans_sklearn.json
 */
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { GO_METRIC_EUCLIDEAN = 0, GO_METRIC_COSINE = 1 };

/* params.cuh:49-99 */
uint32_t go_hash_bitlen(uint32_t beam, uint32_t graph_degree, float max_fill_rate, uint32_t min_bitlen);
uint32_t go_hash_reset_interval(uint32_t beam, uint32_t graph_degree, float max_fill_rate, uint32_t hash_bitlen);
void go_adjust_search_params(uint32_t min_iterations, uint32_t *max_iterations, uint32_t *beam);
/* nn_descent.cuh:1423-1430 */
uint32_t go_nnd_extended_degree(uint32_t degree);
/* utils.cuh:14-19 */
uint32_t go_xorshift32(uint32_t u);

/* bitonic.cuh:24-212; arrays hold M = 32*N elements, element e = N*lane + i */
int go_bitonic_warp_sort(float *keys, uint32_t *vals, uint32_t M);
int go_bitonic_warp_merge(float *keys, uint32_t *vals, uint32_t M, uint32_t range);
/* distance.cuh:29-60 (strided load, blocked store) */
int go_sort_with_key_value(uint32_t max_number, uint32_t number, uint32_t *vals, float *keys);
/* search_kernel.cuh:9-37 and :97-148 on explicit buffers (single-warp variants) */
int go_sort_for_candidate(uint32_t max_cand, float *cand_dist, uint32_t *cand_id, uint32_t degree, uint32_t beam);
int go_sort_for_beam(uint32_t max_beam, float *beam_dist, uint32_t *beam_id, uint32_t beam,
                     const float *cand_dist, const uint32_t *cand_id, uint32_t degree, int first);

/* hashmap.cuh:23-56; table has 2^bitlen entries; sequential insertion in key order */
void go_hashmap_init(uint32_t *table, uint32_t bitlen);
void go_hashmap_insert_seq(uint32_t *table, uint32_t bitlen, const uint32_t *keys, uint32_t n, uint32_t *flags);

/* distance.cuh:9-27, emulating the 32-lane strided partial sums and the shfl_down tree */
float go_distance(const float *a, const float *b, uint32_t dim, int metric);

/* kernel_config.cuh bucket choice */
uint32_t go_max_candidate(uint32_t degree);                      /* 64/128/256, 0 = unsupported */
uint32_t go_max_beam(uint32_t beam);                             /* 64/128/256/512, 0 = unsupported */
uint32_t go_max_centroid_search(uint32_t centroid_num, uint32_t graph_degree); /* kernel_config.cuh:161-171 */
uint32_t go_max_centroid_partition(uint32_t centroid_num);      /* kernel_config.cuh:224-234 */

/* statistics gathered by the search-like routines (algorithmic traffic accounting) */
typedef struct {
    uint64_t iterations;   /* beam iterations executed (parents expanded incl. the entry) */
    uint64_t rows_scored;  /* data rows distance-evaluated */
    uint64_t graph_rows;   /* graph rows read */
} go_stats;

/* search_kernel.cuh:393-490 */
int go_search(const float *data, uint32_t num, uint32_t dim, const uint32_t *graph, uint32_t graph_degree,
              const float *centroids, uint32_t centroid_num, const uint32_t *start_points,
              const float *queries, uint32_t query_num, uint32_t top_k, uint32_t beam,
              uint32_t max_iterations, uint32_t min_iterations, uint32_t hash_bit, uint32_t hash_reset_interval,
              int metric, uint32_t *result_ids, float *result_dists, go_stats *stats, int threads);

/* partition_kernel.cuh:22-66 with slot ids serialised in point order */
int go_partition_assign(const float *data, uint32_t num, uint32_t dim, const float *centroids,
                        uint32_t centroid_num, float boundary_factor, int metric,
                        uint32_t *segment_indexes /* num*3 */, uint32_t *segment_lengths /* C+1 */,
                        float *nearest_dists /* num*2 or NULL */, int threads);
/* partition_kernel.cuh:68-100 */
void go_reorder(const float *data, uint32_t num, uint32_t dim, const uint32_t *segment_indexes,
                const uint32_t *segment_starts, float *reorder_data, uint32_t *map);

/* graph_kernel.cuh:249-316 (build_kernel) over points [0,num) */
int go_build_subgraph(const float *reorder_data, uint32_t num, uint32_t dim, const uint32_t *knn_graph,
                      uint32_t knn_degree, const uint32_t *map, const uint32_t *segment_starts,
                      const uint32_t *segment_lengths, uint32_t segment_num, const uint32_t *start_points,
                      uint32_t graph_degree, uint32_t beam, uint32_t max_iterations, uint32_t min_iterations,
                      uint32_t hash_bit, uint32_t hash_reset_interval, float relaxant, int metric,
                      uint32_t *graph, go_stats *stats, int threads);
/* graph_kernel.cuh:318-376 (build_boundary_kernel) over points [num, reorder_num) */
int go_build_boundary(const float *reorder_data, uint32_t num, uint32_t reorder_num, uint32_t dim,
                      const uint32_t *knn_graph, uint32_t knn_degree, const uint32_t *map,
                      uint32_t start_point, uint32_t graph_degree, uint32_t beam, uint32_t max_iterations,
                      uint32_t min_iterations, uint32_t hash_bit, uint32_t hash_reset_interval, float relaxant,
                      int metric, uint32_t *graph, go_stats *stats, int threads);
/* graph_kernel.cuh:160-247 on one row */
void go_merge_boundary_row(uint32_t *row, uint32_t graph_degree, const uint32_t *neighbors /* reorder ids */,
                           const uint32_t *map);
/* graph_kernel.cuh:70-143 on an explicit pool (ids local, + segment_start); returns neighbour count */
uint32_t go_prune(const float *data, uint32_t dim, uint32_t segment_start, uint32_t *pool_ids, float *pool_dists,
                  uint32_t pool_size, uint32_t graph_degree, float relaxant, int metric, uint32_t *neighbors);
/* graph_kernel.cuh:378-453 with reverse lists serialised by (column, source) */
void go_reverse_edges(uint32_t *graph, uint32_t num, uint32_t graph_degree);
/* graph_kernel.cuh:580-673 reading a snapshot of the graph */
int go_refine(const float *data, uint32_t num, uint32_t dim, uint32_t *graph, uint32_t graph_degree,
              const float *centroids, uint32_t centroid_num, const uint32_t *start_points, uint32_t beam,
              uint32_t max_iterations, uint32_t min_iterations, uint32_t hash_bit, uint32_t hash_reset_interval,
              float relaxant, int metric, go_stats *stats, int threads);

/* large path: select_segment_kernel search_kernel.cuh:546-607 (every output row initialised to 0xffffffff) */
int go_select_segments(const float *queries, uint32_t query_num, uint32_t dim, const float *centroids,
                       uint32_t centroid_num, uint32_t min_segment_num, float boundary_factor, int metric,
                       uint32_t *segment_ids);
/* search_on_sub_kernel + result_merge search_kernel.cuh:609-765 for one segment (final_* updated in place) */
int go_search_sub(const float *seg_data, uint32_t dim, const uint32_t *seg_graph, uint32_t graph_degree,
                  const uint32_t *seg_map, const float *queries, uint32_t query_num, const uint32_t *segment_ids,
                  uint32_t centroid_num, uint32_t segment_id, uint32_t start_point, uint32_t top_k, uint32_t beam,
                  uint32_t max_iterations, uint32_t min_iterations, uint32_t hash_bit, uint32_t hash_reset_interval,
                  int metric, uint32_t *final_ids, float *final_dists, go_stats *stats, int threads);
/* build_for_large_kernel graph_kernel.cuh:675-728 */
int go_build_segment(const float *seg_data, uint32_t num, uint32_t dim, const uint32_t *knn_graph, uint32_t knn_degree,
                     uint32_t start_point, uint32_t graph_degree, uint32_t beam, uint32_t max_iterations,
                     uint32_t min_iterations, uint32_t hash_bit, uint32_t hash_reset_interval, float relaxant,
                     int metric, uint32_t *graph, go_stats *stats, int threads);
/* refine_for_large_kernel graph_kernel.cuh:730-821 */
int go_refine_segment(const float *seg_data, uint32_t num, uint32_t dim, uint32_t *graph, uint32_t graph_degree,
                      uint32_t start_point, uint32_t beam, uint32_t max_iterations, uint32_t min_iterations,
                      uint32_t hash_bit, uint32_t hash_reset_interval, float relaxant, int metric, go_stats *stats,
                      int threads);

/* nn_descent.cuh:668-1467 (intended algorithm; per-partition local ids), K-wide rows out */
int go_nnd_build(const float *reorder_data, uint32_t reorder_num, uint32_t dim, const uint32_t *segment_starts,
                 const uint32_t *segment_lengths, uint32_t segment_num, uint32_t knn_degree,
                 uint32_t iterations, uint32_t seed, int32_t *knn_graph, int threads);

/* the same with NNDescentParameter::termination_threshold (params.cuh:21; update counter nn_descent.cuh:1123,1270-1284) */
int go_nnd_build_ex(const float *reorder_data, uint32_t reorder_num, uint32_t dim, const uint32_t *segment_starts,
                    const uint32_t *segment_lengths, uint32_t segment_num, uint32_t knn_degree, uint32_t iterations,
                    float termination_threshold, uint32_t seed, int32_t *knn_graph, int threads);
/* The same build with the host loop as the reference ships it (length passed as end, partition-local id compared with the
 * global row index, no merge across sub-lists before truncation; nn_descent.cuh:1276-1283, :1117, :1376-1402).  Only
 * for quoting what the shipped executable would score; nothing is held to it. */
/* go_nnd_build_ex from start lists the caller brings (reorder_num x extended degree partition-local ids, a row's sub-lists
 * one after the other, negative = empty) instead of the shuffled ones of init_random_graph (nn_descent.cuh:1003-1038):
 * lets a test start both sides of a comparison from one random graph. */
int go_nnd_build_from(const float *reorder_data, uint32_t reorder_num, uint32_t dim, const uint32_t *segment_starts,
                      const uint32_t *segment_lengths, uint32_t segment_num, uint32_t knn_degree, uint32_t iterations,
                      float termination_threshold, const int32_t *start_lists, int32_t *knn_graph, int threads);
int go_nnd_build_shipped(const float *reorder_data, uint32_t reorder_num, uint32_t dim, const uint32_t *segment_starts,
                         const uint32_t *segment_lengths, uint32_t segment_num, uint32_t knn_degree, uint32_t iterations,
                         float termination_threshold, uint32_t seed, int32_t *knn_graph, int threads);

/* exact kNN by brute force (ties by smaller id); squared L2 ranking, reported per metric */
void go_bruteforce_knn(const float *data, uint32_t num, uint32_t dim, const float *queries, uint32_t query_num,
                       uint32_t k, int metric, int exclude_self, uint32_t *ids, float *dists, int threads);
/* Lloyd k-means (stand-in for cuvs::cluster::kmeans::fit, partition.cuh:48-54) */
void go_kmeans_seed(const float *sample, uint32_t n, uint32_t dim, uint32_t k, uint32_t seed, float *centroids,
                    uint32_t *chosen_out);
void go_kmeans_from(const float *sample, uint32_t n, uint32_t dim, uint32_t k, uint32_t iterations, float *centroids);
void go_kmeans(const float *sample, uint32_t n, uint32_t dim, uint32_t k, uint32_t iterations, uint32_t seed,
               float *centroids);

#ifdef __cplusplus
}
#endif
