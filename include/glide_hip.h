/*
 * glide_hip.h -- C ABI of the MI355X (gfx950) GLIDE kernels.
 *
 * Every entry point takes raw device pointers and plain sizes, launches on `stream` (a hipStream_t passed as
 * void*, NULL = default stream) and returns an int: 0 = success, > 0 = a hipError_t value, < 0 = one of the
 * GLIDE_ERR_* argument errors below.  No exceptions cross the boundary and the library keeps no global state apart
 * from the scratch array of glide_hip_partition_assign_fixed.
 * Each declaration cites the interface of the reference implementation (owlet-hub/GLIDE, paths relative to its
 * src/ directory) that it replaces.
 *
 * No entry point allocates device memory: those that need scratch take a caller-provided `workspace` whose
 * size a companion *_workspace_bytes() function reports (glide_hip_partition_assign_fixed brings its own).
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
#define GLIDE_COUNTER_STRIPES 256

/* ---- library / device ------------------------------------------------------------------------------------ */
const char *glide_hip_version(void);
const char *glide_hip_error_string(int code);
/* replaces the hard-coded cudaSetDevice(1) of the reference mains (small_build.cu:33) */
int glide_hip_set_device(int device);
int glide_hip_device_info(char *name, size_t name_len, int *compute_units, size_t *total_mem);
/* free and total device memory of the current device (hipMemGetInfo); no counterpart in the reference: lets a host
 * size its staging buffers and lets a test see that an entry point allocates nothing */
int glide_hip_mem_info(size_t *free_bytes, size_t *total_bytes);

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
 * query_num x top_k.  `counters` (nullable) points at GLIDE_COUNTER_STRIPES x 3 u64 that the caller zeroed; the
 * kernel adds {beam iterations, data rows scored, graph rows read} into the stripe of each workgroup (one shared
 * address would serialise the launch); the sums over the stripes are the algorithmic-traffic tallies.
 * Limits (reference kernel_config.cuh:41-60): graph_degree <= 256, beam <= 512, centroid_num <= 256, dim % 4 == 0,
 * dim <= 4096, top_k <= beam; a beam above 256 is a multiple of 16 (params.cuh:82-99 rounds beams to multiples of 32).
 * Degrees above 128 and beams above 256 run the candidate sort / beam merge as two half-wave networks, as the
 * reference's two-warp branches do (search_kernel.cuh:38-94, :149-232). */
int glide_hip_search(const float *data, uint32_t num, uint32_t dim, const uint32_t *graph, uint32_t graph_degree,
                     const float *centroids, uint32_t centroid_num, const uint32_t *start_points,
                     const float *queries, uint32_t query_num, uint32_t top_k, uint32_t beam,
                     uint32_t max_iterations, uint32_t min_iterations, uint32_t hash_bit,
                     uint32_t hash_reset_interval, int metric, uint32_t *result_ids, float *result_dists,
                     unsigned long long *counters, void *stream);

/* ---- locality partitioning (subsystem 1) --------------------------------------------------------------------
 * Replaces define_partition_kernel (partition_kernel.cuh:22-66) + the host prefix sum of define_partition
 * (partition.cuh:61-116).  Distances to all centroids are ranked with an fp32 MFMA tile (||c||^2 - 2 x.c), the
 * best four are re-evaluated with the direct sum of squared differences, and the reference's rule is applied to
 * those: segment = nearest centroid; boundary iff centroid_num > 1 and d(2nd)/d(1st) <= boundary_factor (sqrt
 * distances for Euclidean).  segment_indexes is num x 3: {segment, slot in segment, boundary slot or
 * 0xffffffff}.  Slots are numbered in point order (the reference numbers them in atomicAdd arrival order).
 * segment_lengths receives centroid_num + 1 counts, the last one being the boundary list.  nearest_dists
 * (nullable, num x 2) receives the two smallest distances.  Limits: centroid_num <= 256, dim % 4 == 0. */
size_t glide_hip_partition_assign_workspace_bytes(uint32_t num, uint32_t centroid_num);
int glide_hip_partition_assign(const float *data, uint32_t num, uint32_t dim, const float *centroids,
                               uint32_t centroid_num, float boundary_factor, int metric,
                               uint32_t *segment_indexes, uint32_t *segment_lengths, float *nearest_dists,
                               void *workspace, size_t workspace_bytes, void *stream);

/* glide_hip_partition_assign without a workspace argument.  No counterpart in the reference: it is for callers that
 * cannot allocate device memory (code under HIP graph capture, serving loops that route batches of new points or
 * queries to their partitions, harnesses that forbid hipMalloc).  The scratch memory (centroid norms + per-tile
 * histograms, 515 KB) is a file-scope device array of the library; each GPU the library runs on holds it until the
 * process ends.  At most glide_hip_partition_assign_fixed_max_points() = 65536 points per call (GLIDE_ERR_UNSUPPORTED
 * beyond); other limits, arguments and results as glide_hip_partition_assign.  The call allocates and frees nothing.
 * The array's device address is looked up on the first call on each device (not a stream operation: make that
 * first call outside a capture).  All calls on one GPU share the array: calls that overlap on one GPU (different
 * streams or threads) race and must be serialised by the caller. */
uint32_t glide_hip_partition_assign_fixed_max_points(void);
int glide_hip_partition_assign_fixed(const float *data, uint32_t num, uint32_t dim, const float *centroids,
                                     uint32_t centroid_num, float boundary_factor, int metric,
                                     uint32_t *segment_indexes, uint32_t *segment_lengths, float *nearest_dists,
                                     void *stream);

/* Replaces reorder_kernel (partition_kernel.cuh:68-100; partition.cuh:118-157): row p goes to
 * segment_starts[segment] + slot, boundary copies to num + boundary slot; map[reorder id] = p.
 * segment_starts: centroid_num + 1 device words (exclusive prefix sum of segment_lengths). */
int glide_hip_reorder(const float *data, uint32_t num, uint32_t dim, const uint32_t *segment_indexes,
                      const uint32_t *segment_starts, float *reorder_data, uint32_t *map, void *stream);

/* Batched form for data sets staged through the GPU in pieces (replaces reorder_for_large_kernel,
 * partition_kernel.cuh:164-193; partition.cuh:339-415): `data` holds `num` rows of one batch, segment_starts the
 * offsets of the segments inside this batch's output buffer, and map receives point_id_offset + row. */
int glide_hip_reorder_batch(const float *data, uint32_t num, uint32_t dim, const uint32_t *segment_indexes,
                            const uint32_t *segment_starts, uint32_t point_id_offset, float *reorder_data,
                            uint32_t *map, void *stream);

/* Replaces sample_kernel (partition_kernel.cuh:7-20; partition.cuh:31-45): sample[i] = data[sample_ids[i]]. */
int glide_hip_sample_rows(const float *data, uint32_t dim, const uint32_t *sample_ids, uint32_t sample_num,
                          float *sample, void *stream);

/* Stands in for cuvs::cluster::kmeans::fit (third-party, rapidsai/cuvs 24.08; call site partition.cuh:48-54) in two
 * calls.  glide_hip_kmeans_seed: greedy k-means++ seeding.  Every further centroid is the best of 2 + floor(ln k)
 * sample rows drawn with probability proportional to their squared distance from the nearest centroid chosen so
 * far, best = smallest remaining potential (cuVS initialises with its k-means++ family by default).  The draws are a
 * hash of (seed, step, trial), so a run is reproducible.  chosen_rows (nullable, cluster_num u32) receives the sample
 * rows taken.  workspace: 8-byte aligned.  glide_hip_kmeans_fit: `iterations` Lloyd steps from the centroids passed in;
 * the cluster sums are accumulated in 64-bit fixed point, so a fit is reproducible bit for bit (workspace: 8-byte aligned). */
size_t glide_hip_kmeans_seed_workspace_bytes(uint32_t sample_num);
int glide_hip_kmeans_seed(const float *sample, uint32_t sample_num, uint32_t dim, uint32_t cluster_num, uint32_t seed,
                          float *centroids, uint32_t *chosen_rows, void *workspace, size_t workspace_bytes,
                          void *stream);
size_t glide_hip_kmeans_workspace_bytes(uint32_t cluster_num, uint32_t dim);
int glide_hip_kmeans_fit(const float *sample, uint32_t sample_num, uint32_t dim, uint32_t cluster_num,
                         uint32_t iterations, float *centroids, void *workspace, size_t workspace_bytes,
                         void *stream);

/* ---- NN-descent kNN graph (subsystem 2) ---------------------------------------------------------------------
 * Replaces build_nnd / GNND::build (nn_descent.cuh:1238-1467) together with its device kernels
 * (preprocess_data_kernel :445, add_rev_edges_kernel :490, local_join_kernel :668) and the host-side sampling
 * and list merging (GnndGraph :973-1149).  Builds, for every partition given by segment_starts/segment_lengths
 * (device arrays, segment_num entries, the boundary segment included), a knn_degree-regular graph of
 * partition-local ids: knn_graph is reorder_num x knn_degree, nearest first.  `iterations` rounds of
 * sample -> reverse sample -> local join (64 x 64 fp16 matrix-core tiles, fp32 accumulate, norm-trick
 * epilogue, one offer per row/column) -> merge are run; lists, flags and samples stay in `workspace`.
 * termination_threshold (NNDescentParameter::termination_threshold, params.cuh:21; 0 disables): a partition whose
 * list insertions on every 100th row fall below termination_threshold * reorder_num * dim / 100 in a round
 * (nn_descent.cuh:1123,1280) runs one more round and is then left alone; from the third round on the partition
 * states are read back after each round (the call then waits on `stream`) and the loop ends once every partition
 * rests.  At most 2048 partitions.
 * stats_out (nullable, 2 device u64): distinct offers the merge steps found in the offer tables; offers that stayed
 * away because their target had announced a distance threshold (see `offers` and `norms` below).
 * Limits: knn_degree <= 256, the widest degree the build searches that read the kNN graph take (list width
 * round_up32(1.3 * knn_degree) <= 352 = eleven sub-lists, Bloom filter <= 8192 bits),
 * dim % 4 == 0, reorder_num < 2^26 and reorder_num * list width < 2^32 per call (the large path calls it partition by
 * partition).  Two builds with the same inputs and seed give the same graph: nothing depends on the order in which
 * atomic operations arrive. */
size_t glide_hip_nnd_workspace_bytes(uint32_t reorder_num, uint32_t dim, uint32_t knn_degree);
int glide_hip_nnd_build(const float *reorder_data, uint32_t reorder_num, uint32_t dim,
                        const uint32_t *segment_starts, const uint32_t *segment_lengths, uint32_t segment_num,
                        uint32_t knn_degree, uint32_t iterations, float termination_threshold, uint32_t seed,
                        uint32_t *knn_graph, void *workspace, size_t workspace_bytes, unsigned long long *stats_out,
                        void *stream);

/* The same build one stage per call, on the same workspace (the stages of GNND::build's loop, nn_descent.cuh:1289-1368):
 *   prepare         preprocess_data_kernel :445 (fp16 rows + fp32 squared norms), init_random_graph :1003,
 *                   Bloom filter cleared, first samples (sample_graph(true) :1040-1071)
 *   reverse_sample  add_rev_edges_kernel :490-507
 *   local_join      local_join_kernel :668-914; offers go to the per-node offer table instead of a spin-locked
 *                   list; it restarts the reverse lists it has read
 *   merge           update_graph :1106-1126 + sample_graph_new :973-1001 + sample_segment_graph :1073-1104
 *   converge        the termination test of update_and_sample :1270-1284 (marks partitions that rest from now on)
 *   finalize        the shrink step :1376-1402
 *   sample          sample_graph :1040-1071 on its own (prepare and merge include it)
 * glide_hip_nnd_build = prepare, `iterations` x (reverse_sample, local_join, merge, converge), finalize.
 * glide_hip_nnd_layout reports where each array lives in the workspace (byte offsets), so a caller or a test can
 * inspect or replace any of them between stages:
 *   list_ids   num x width u32: partition-local id | 0x80000000 ("already sampled"), 0xffffffff = empty.  width / 32
 *                   sub-lists keyed by id % (width / 32), each nearest first; entry r of sub-list s is slot
 *                   r * (width / 32) + s (the order in which the reference samples, nn_descent.cuh:1052-1068)
 *   list_dists num x width f32 (squared L2 of the fp16 rows, FLT_MAX for the random start entries)
 *   fwd_new / fwd_old  num x 32 u32 sample lists, rev_new / rev_old  num rows of reverse_stride (72) u32 holding up to
 *                   reverse_cap (64) reverse samples in order of arrival; counts num x 4 u32 = their lengths (the reverse lengths count every arrival and may exceed
 *                   reverse_cap; the join uses the 32 smallest)
 *   members    num x 128 u32 and member_counts num x 2 u32: the lists a join works on, written by local_join before its
 *                   tiles: slots 0..63 the new members (forward samples, then the 32 smallest reverse sources, duplicates
 *                   removed), slots 64..127 the old ones; slots beyond the counts keep what an earlier round left there
 *   offers     num x offer_slots u64 keys (distance bits << 32 | candidate id, all ones = empty): the offers of the
 *                   round.  offer_slots is 256 when the list is one sub-list (knn_degree <= 32) and 512 otherwise.  With
 *                   x = candidate ^ round * 0x85EBCA6B, an offer goes to slot s1 = (x * 0x9E3779B1) >> (32 - log2
 *                   offer_slots) of its target's row and to a second slot of the same 16-slot line,
 *                   (s1 & ~15) | ((s1 + 1 + umulhi(x * 0xC2B2AE35, 15)) & 15), and stays in each where it is the
 *                   smallest key the slot has seen (an atomic minimum): copies of one offer fall together, of two
 *                   candidates that share a slot the nearer one stays.  The merge reads the row, uses its 32 smallest
 *                   distinct keys and empties it.  `round` (one u32, raised by converge) changes the slots from round
 *                   to round.
 *   rev_tables num x 2 (new, old) x reverse_slots (256) u32: overflow tables for what arrives after a reverse list is
 *                   full.  They are made of buckets of 16 words: 15 slots (all ones = empty, slot order is a hash
 *                   order) and, last, the bucket's bound = the smallest key it has turned away (all ones: none).  A
 *                   key's bucket is the top 4 bits of id * 0x9E3779B1; a bucket keeps the 15 smallest distinct keys sent
 *                   to it.  The join uses the 32 smallest sources of list + table.
 *   norms      num x (f32 squared norm of the fp32 row, u32 offer threshold); rev_thr num x 2 u32.  Thresholds are
 *                   what a crowded node announces for the next round (an offer table with five eighths of its slots taken:
 *                   the distance bits of its 64th smallest key; a reverse list that overflowed: its 56th smallest source):
 *                   offers whose distance bits (sources whose ids) are not below it stay away; all ones = none.  None
 *                   of this depends on the order in which atomic operations arrive.
 *   bloom      num x bloom_sets x 512 bits
 *   segment_state   u32 per partition: 0 active, 1 last round, 2 resting;  segment_updates  u32 per partition */
typedef struct {
    uint64_t half_rows, norms, list_ids, list_dists, fwd_new, fwd_old, rev_new, rev_old, rev_tables, rev_thr, counts,
        members, member_counts, offers, bloom, segment_state, segment_updates, round, total;
    uint32_t width, reverse_cap, reverse_stride, offer_slots, reverse_slots, row_halfs, bloom_sets, reserved;
} glide_nnd_layout;
int glide_hip_nnd_layout(uint32_t reorder_num, uint32_t dim, uint32_t knn_degree, glide_nnd_layout *out);
int glide_hip_nnd_prepare(const float *reorder_data, uint32_t reorder_num, uint32_t dim, const uint32_t *segment_starts,
                          const uint32_t *segment_lengths, uint32_t segment_num, uint32_t knn_degree, uint32_t seed,
                          void *workspace, size_t workspace_bytes, void *stream);
/* sample_graph (nn_descent.cuh:1040-1071) on the lists as they stand: per list the first <= 32 entries not yet flagged
 * become its new samples and are flagged, the first <= 32 flagged ones its old samples; the reverse counts restart.
 * prepare has already done this for the start lists and merge does it for every later round, so the build loop never
 * calls it; it is there for a caller that replaces the lists between stages. */
int glide_hip_nnd_sample(uint32_t reorder_num, uint32_t dim, const uint32_t *segment_starts,
                         const uint32_t *segment_lengths, uint32_t segment_num, uint32_t knn_degree, void *workspace,
                         size_t workspace_bytes, void *stream);
int glide_hip_nnd_reverse_sample(uint32_t reorder_num, uint32_t dim, const uint32_t *segment_starts,
                                 const uint32_t *segment_lengths, uint32_t segment_num, uint32_t knn_degree,
                                 void *workspace, size_t workspace_bytes, void *stream);
int glide_hip_nnd_local_join(uint32_t reorder_num, uint32_t dim, const uint32_t *segment_starts,
                             const uint32_t *segment_lengths, uint32_t segment_num, uint32_t knn_degree,
                             void *workspace, size_t workspace_bytes, void *stream);
int glide_hip_nnd_merge(uint32_t reorder_num, uint32_t dim, const uint32_t *segment_starts,
                        const uint32_t *segment_lengths, uint32_t segment_num, uint32_t knn_degree,
                        void *workspace, size_t workspace_bytes, void *stream);
int glide_hip_nnd_converge(uint32_t reorder_num, uint32_t dim, const uint32_t *segment_starts,
                           const uint32_t *segment_lengths, uint32_t segment_num, uint32_t knn_degree,
                           float termination_threshold, void *workspace, size_t workspace_bytes, void *stream);
int glide_hip_nnd_finalize(uint32_t reorder_num, uint32_t dim, const uint32_t *segment_starts,
                           const uint32_t *segment_lengths, uint32_t segment_num, uint32_t knn_degree,
                           uint32_t *knn_graph, unsigned long long *stats_out, void *workspace, size_t workspace_bytes,
                           void *stream);

/* ---- graph construction (subsystem 3) ----------------------------------------------------------------------
 * All kernels give one point to one wavefront.  Limits as for glide_hip_search (knn_degree, graph_degree <= 256,
 * beam <= 512, dim % 4 == 0, dim <= 4096).  `counters` as in glide_hip_search (prune distances count as rows). */

/* Replaces build_kernel (graph_kernel.cuh:249-316) as launched by GLIDE::subgraph_build_and_merge
 * (glide_impl.cuh:77-147): for every reorder id p < num, beam search on the partition-local kNN graph from the
 * partition's start point, relaxed-RNG prune to graph_degree, row graph[map[p]] written in original ids
 * (0xffffffff = empty).  knn_graph is reorder_num x knn_degree with partition-local ids; start_points holds one
 * partition-local id per segment. */
int glide_hip_build_subgraph(const float *reorder_data, uint32_t num, uint32_t dim, const uint32_t *knn_graph,
                             uint32_t knn_degree, const uint32_t *map, const uint32_t *segment_starts,
                             const uint32_t *segment_lengths, uint32_t segment_num, const uint32_t *start_points,
                             uint32_t graph_degree, uint32_t beam, uint32_t max_iterations,
                             uint32_t min_iterations, uint32_t hash_bit, uint32_t hash_reset_interval,
                             float relaxant, int metric, uint32_t *graph, unsigned long long *counters,
                             void *stream);

/* Replaces build_boundary_kernel + map_to_graph_boundary (graph_kernel.cuh:318-376, 160-247; launch
 * glide_impl.cuh:149-191): the same on the boundary segment [num, reorder_num), merging each result into the
 * row of the original point.  Must run after glide_hip_build_subgraph on the same stream.  start_point is the
 * boundary segment's local start id. */
int glide_hip_build_boundary(const float *reorder_data, uint32_t num, uint32_t reorder_num, uint32_t dim,
                             const uint32_t *knn_graph, uint32_t knn_degree, const uint32_t *map,
                             uint32_t start_point, uint32_t graph_degree, uint32_t beam, uint32_t max_iterations,
                             uint32_t min_iterations, uint32_t hash_bit, uint32_t hash_reset_interval,
                             float relaxant, int metric, uint32_t *graph, unsigned long long *counters,
                             void *stream);

/* Replaces the graph_degree launches of reverse_graph_kernel (graph_kernel.cuh:378-414; glide_impl.cuh:194-233).
 * reverse_graph (num x graph_degree) receives, for every node, the sources of edges pointing at it that it does
 * not point back to, capped at graph_degree; reverse_counts the uncapped count.  Where the reference keeps
 * whichever sources win its atomics, the list here is the first graph_degree in (column, source) order, i.e.
 * what a sequential sweep produces.  workspace: glide_hip_reverse_edges_workspace_bytes(), 8-byte aligned. */
size_t glide_hip_reverse_edges_workspace_bytes(uint32_t num, uint32_t graph_degree);
int glide_hip_reverse_edges(const uint32_t *graph, uint32_t num, uint32_t graph_degree, uint32_t *reverse_graph,
                            uint32_t *reverse_counts, void *workspace, size_t workspace_bytes, void *stream);

/* Replaces insert_reverse_kernel (graph_kernel.cuh:416-453; glide_impl.cuh:235-256): the empty slots of each
 * row take, in order, the first entries of its reverse list. */
int glide_hip_insert_reverse(uint32_t *graph, const uint32_t *reverse_graph, const uint32_t *reverse_counts,
                             uint32_t num, uint32_t graph_degree, void *stream);

/* Replaces refine_kernel (graph_kernel.cuh:580-673; GLIDE::refine glide_impl.cuh:258-316): rows with empty
 * slots search the whole graph from the nearest centroid's start point and fill the slots after a prune that
 * skips existing neighbours.  Reads graph_in, writes every row of graph_out (graph_in != graph_out): the
 * reference refines in place while other blocks still traverse the rows; here all searches see the
 * pre-refinement graph.  `order` (nullable) is a permutation of the points: workgroup i refines point order[i].  The
 * result does not depend on it; handing in the partition order (the first `num` entries of `map`) makes wavefronts
 * that run together search the same region, which cuts HBM traffic (1M x 128 mixture data: 0.168 s -> 0.109 s). */
int glide_hip_refine(const float *data, uint32_t num, uint32_t dim, const uint32_t *graph_in, uint32_t *graph_out,
                     uint32_t graph_degree, const float *centroids, uint32_t centroid_num,
                     const uint32_t *start_points, uint32_t beam, uint32_t max_iterations,
                     uint32_t min_iterations, uint32_t hash_bit, uint32_t hash_reset_interval, float relaxant,
                     int metric, const uint32_t *order, unsigned long long *counters, void *stream);

/* ---- large path: one staged partition at a time (GLIDE_large, glide_large_impl.cuh) ---------------------------
 * The partition's rows, kNN graph / graph and map are device arrays holding only that partition (ids are
 * partition-local); the caller stages them (the reference copies each partition from host memory,
 * glide_large_impl.cuh:109-166).  Data type: float (the reference's large executables instantiate uint8). */

/* Queries grouped by the partitions they selected (no counterpart in the reference, whose search_on_sub_kernel starts
 * one block per query of the batch for every partition and lets the blocks of other partitions return at once).
 * segment_ids: query_num x centroid_num from glide_hip_select_segments.  counts (centroid_num u32) and offsets
 * (centroid_num + 1 u32) describe lists (at most query_num x centroid_num u32): the queries that selected partition
 * s are lists[offsets[s] .. offsets[s + 1]), in no particular order.  All device arrays. */
size_t glide_hip_group_queries_workspace_bytes(uint32_t centroid_num);
int glide_hip_group_queries(const uint32_t *segment_ids, uint32_t query_num, uint32_t centroid_num, uint32_t *counts,
                            uint32_t *offsets, uint32_t *lists, void *workspace, size_t workspace_bytes, void *stream);

/* glide_hip_search_sub for the queries named in query_list (list_len of them) instead of a scan of segment_ids. */
int glide_hip_search_sub_listed(const float *segment_data, uint32_t dim, const uint32_t *segment_graph,
                                uint32_t graph_degree, const uint32_t *segment_map, const float *queries,
                                uint32_t query_num, const uint32_t *query_list, uint32_t list_len, uint32_t segment_id,
                                uint32_t start_point, uint32_t top_k, uint32_t beam, uint32_t max_iterations,
                                uint32_t min_iterations, uint32_t hash_bit, uint32_t hash_reset_interval, int metric,
                                uint32_t *final_ids, float *final_dists, unsigned long long *counters, void *stream);

/* The whole per-partition search of GLIDE_large::search (glide_large_impl.cuh:347-507) on an index resident in device
 * memory, in three launches instead of one per partition: the queries are grouped by partition, one wavefront per
 * (query, selected partition) pair runs search_on_sub_kernel's search and leaves the head of its beam, and one
 * wavefront per query merges its heads in ascending partition order, the order of the partition-by-partition loop,
 * so ids and distances are the same.  data / graph / map hold all partitions in reorder order (graph ids are
 * partition-local); segment_starts and segment_start_points (local; 0xffffffff marks an empty partition) are device
 * arrays of segment_num entries;
 * segment_ids comes from glide_hip_select_segments with centroid_num = segment_num.  final_ids / final_dists
 * (query_num x top_k) are overwritten.  The call waits on `stream` once (it reads the number of pairs back).
 * workspace: glide_hip_search_partitions_workspace_bytes(), sized for every query selecting every partition. */
size_t glide_hip_search_partitions_workspace_bytes(uint32_t query_num, uint32_t centroid_num, uint32_t top_k);
int glide_hip_search_partitions(const float *data, uint32_t dim, const uint32_t *graph, uint32_t graph_degree,
                                const uint32_t *map, const uint32_t *segment_starts,
                                const uint32_t *segment_start_points, uint32_t segment_num, const float *queries,
                                uint32_t query_num, const uint32_t *segment_ids, uint32_t top_k, uint32_t beam,
                                uint32_t max_iterations, uint32_t min_iterations, uint32_t hash_bit,
                                uint32_t hash_reset_interval, int metric, uint32_t *final_ids, float *final_dists,
                                void *workspace, size_t workspace_bytes, unsigned long long *counters, void *stream);

/* ---- merged large build (GLIDE_large::build_with_merge, declared at glide_large.cuh:89-97 without a definition) --
 * The merged graph lives in device memory in reorder-id space: row r belongs to reorder row r (r < num) and holds
 * reorder ids.  The two passes below are the large-path forms of map_to_graph (graph_kernel.cuh:145-150) and
 * map_to_graph_boundary (graph_kernel.cuh:160-247), which the small path runs fused into its build kernels. */

/* glide_hip_search on a merged large index.  The only difference: every centroid is ranked to pick the entry point
 * (the bucket of the centroid sort comes from centroid_num), where glide_hip_search takes the bucket from
 * graph_degree as the reference's small path does (kernel_config.cuh:161-171) and so ranks at most the first 64
 * centroids of a degree-32 index; a large index has up to 256 partitions. */
int glide_hip_search_merged(const float *data, uint32_t num, uint32_t dim, const uint32_t *graph, uint32_t graph_degree,
                            const float *centroids, uint32_t centroid_num, const uint32_t *start_points,
                            const float *queries, uint32_t query_num, uint32_t top_k, uint32_t beam,
                            uint32_t max_iterations, uint32_t min_iterations, uint32_t hash_bit,
                            uint32_t hash_reset_interval, int metric, uint32_t *result_ids, float *result_dists,
                            unsigned long long *counters, void *stream);

/* glide_hip_refine on a merged large graph: as glide_hip_refine, every centroid ranked for the entry point (see
 * glide_hip_search_merged). */
int glide_hip_refine_merged(const float *data, uint32_t num, uint32_t dim, const uint32_t *graph_in, uint32_t *graph_out,
                            uint32_t graph_degree, const float *centroids, uint32_t centroid_num,
                            const uint32_t *start_points, uint32_t beam, uint32_t max_iterations,
                            uint32_t min_iterations, uint32_t hash_bit, uint32_t hash_reset_interval, float relaxant,
                            int metric, const uint32_t *order, unsigned long long *counters, void *stream);

/* Rows of one staged partition's sub-graph (partition-local ids, from glide_hip_build_segment) go to rows
 * segment_start.. of the merged graph, every id shifted by segment_start; empty slots stay 0xffffffff. */
int glide_hip_place_segment_graph(const uint32_t *segment_graph, uint32_t segment_length, uint32_t graph_degree,
                                  uint32_t segment_start, uint32_t *merged_graph, void *stream);

/* boundary_graph (boundary_num x graph_degree, ids local to the boundary segment) is the sub-graph built over the
 * boundary copies.  Copy i is merged into merged_graph row home_rows[i] (the row of the point it duplicates) by the
 * rule of map_to_graph_boundary, a neighbour l being entered as home_rows[l].  No two copies share a home row. */
int glide_hip_merge_boundary_graph(const uint32_t *boundary_graph, uint32_t boundary_num, uint32_t graph_degree,
                                   const uint32_t *home_rows, uint32_t *merged_graph, void *stream);

/* Replaces build_for_large_kernel (graph_kernel.cuh:675-728; launch glide_large_impl.cuh:140): sub-graph of one
 * partition, rows written with partition-local ids. */
int glide_hip_build_segment(const float *segment_data, uint32_t num, uint32_t dim, const uint32_t *knn_graph,
                            uint32_t knn_degree, uint32_t start_point, uint32_t graph_degree, uint32_t beam,
                            uint32_t max_iterations, uint32_t min_iterations, uint32_t hash_bit,
                            uint32_t hash_reset_interval, float relaxant, int metric, uint32_t *graph,
                            unsigned long long *counters, void *stream);
/* Replaces refine_for_large_kernel (graph_kernel.cuh:730-821; launch glide_large_impl.cuh:303): as
 * glide_hip_refine, searching from the partition's start point. */
int glide_hip_refine_segment(const float *segment_data, uint32_t num, uint32_t dim, const uint32_t *graph_in,
                             uint32_t *graph_out, uint32_t graph_degree, uint32_t start_point, uint32_t beam,
                             uint32_t max_iterations, uint32_t min_iterations, uint32_t hash_bit,
                             uint32_t hash_reset_interval, float relaxant, int metric,
                             unsigned long long *counters, void *stream);
/* Replaces select_segment_kernel (search_kernel.cuh:546-607; launch glide_large_impl.cuh:408): segment_ids is
 * query_num x centroid_num; row q lists the partitions query q visits (nearest first: those whose centroid
 * distance is within boundary_factor of the nearest, topped up to min_segment_num), then 0xffffffff. */
int glide_hip_select_segments(const float *queries, uint32_t query_num, uint32_t dim, const float *centroids,
                              uint32_t centroid_num, uint32_t min_segment_num, float boundary_factor, int metric,
                              uint32_t *segment_ids, void *stream);
/* Replaces search_on_sub_kernel + result_merge (search_kernel.cuh:609-765; launch glide_large_impl.cuh:468): queries
 * that list `segment_id` search the staged partition and merge its best top_k (mapped to original ids through
 * segment_map) into final_ids / final_dists (query_num x top_k, initialised by the caller to 0xffffffff /
 * FLT_MAX before the first partition).  Limits as glide_hip_search, top_k <= 128. */
int glide_hip_search_sub(const float *segment_data, uint32_t dim, const uint32_t *segment_graph,
                         uint32_t graph_degree, const uint32_t *segment_map, const float *queries,
                         uint32_t query_num, const uint32_t *segment_ids, uint32_t centroid_num,
                         uint32_t segment_id, uint32_t start_point, uint32_t top_k, uint32_t beam,
                         uint32_t max_iterations, uint32_t min_iterations, uint32_t hash_bit,
                         uint32_t hash_reset_interval, int metric, uint32_t *final_ids, float *final_dists,
                         unsigned long long *counters, void *stream);
/* asynchronous copies for staging (the caller orders them with streams / events; host memory should be pinned) */
int glide_hip_memcpy_h2d_async(void *dst, const void *src, size_t bytes, void *stream);
int glide_hip_memcpy_d2h_async(void *dst, const void *src, size_t bytes, void *stream);
int glide_hip_stream_wait_event(void *stream, void *event);

/* uint8 rows -> fp32 rows on the device (count values; src 4-byte aligned, dst 16-byte aligned).  The reference's large
 * path keeps uint8 rows and casts each byte to float where a kernel reads it (search_kernel.cuh:493-544,
 * graph_kernel.cuh:675-821); here a staged partition is widened once after its upload and every kernel reads fp32. */
int glide_hip_widen_u8(const unsigned char *src, size_t count, float *dst, void *stream);

/* Rows of src_dim values -> rows of dst_dim values: the first min(src_dim, dst_dim) values of every row, zeros behind
 * them (both 4-byte aligned, no overlap).  Every other entry point reads rows in 16-byte pieces and wants dim % 4 == 0;
 * the reference's kernels loop over single values and take any dim (distance.cuh:9-27).  Points of another length are
 * padded once with this call (dst_dim = dim rounded up to a multiple of 4; a zero coordinate changes no squared
 * distance, inner product or norm) and centroids or reordered rows are cut back with it where a caller wants them. */
int glide_hip_copy_rows(const float *src, uint64_t num, uint32_t src_dim, float *dst, uint32_t dst_dim, void *stream);

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
