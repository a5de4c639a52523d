// The large path's search: partitions ranked per query, queries grouped by partition, a beam search inside each staged
// partition and the running merge of the per-partition results.
// Reference: select_segment_kernel (search_kernel.cuh:546-607), search_on_sub_kernel (:653-765) with result_merge (:609-651),
// as launched by GLIDE_large::search (glide_large_impl.cuh:347-507).
#include "beam.hpp"
#include "host_util.hpp"

namespace glide {

// ---- large path: one staged partition at a time ---------------------------------------------------------------
// select_segment_kernel (search_kernel.cuh:546-607): rank the centroids for each query; keep those within
// boundary_factor of the nearest, topped up to min_segment_num.  Unlike the reference, which resets only the first
// output row and leaves the rest uninitialised, every row starts as 0xffffffff.
struct SelectArgs {
    const float* queries;
    const float* centroids;
    uint32_t* segment_ids;
    uint32_t query_num, dim, centroid_num, min_segment_num;
    float boundary_factor;
    int metric;
};

template <int MAX_CENTROID>
__global__ __launch_bounds__(64) void select_segments_kernel(SelectArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    float* cent_dist = reinterpret_cast<float*>(smem);
    uint32_t* cent_id = reinterpret_cast<uint32_t*>(cent_dist + round_up32(a.centroid_num));
    const uint32_t q = blockIdx.x;
    if (q >= a.query_num) return;
    const int lane = lane_id();
    const int half = lane >> 5, t = lane & 31;
    const float* query = a.queries + static_cast<size_t>(q) * a.dim;
    for (uint32_t c0 = 0; c0 < a.centroid_num; c0 += 2) {
        const uint32_t c = c0 + half < a.centroid_num ? c0 + half : c0;
        float acc = 0.f;
        for (uint32_t d0 = t * 4; d0 < a.dim; d0 += 128) {
            acc = sqdist4(*reinterpret_cast<const float4*>(query + d0),
                          *reinterpret_cast<const float4*>(a.centroids + static_cast<size_t>(c) * a.dim + d0), acc);
        }
        const float d = finish_distance(half_wave_sum(acc), a.metric);
        if (t == 0 && c0 + half < a.centroid_num) cent_dist[c0 + half] = d;
    }
    wave_sync();
    constexpr int NR = WaveNet<MAX_CENTROID>::NR;
    constexpr int N32 = MAX_CENTROID / 32;
    float k[NR];
    uint32_t v[NR];
#pragma unroll
    for (int r = 0; r < NR; r++) {
        const uint32_t e = NR * lane + r;
        const uint32_t j = (e / N32) + 32 * (e % N32);
        const bool ok = (MAX_CENTROID >= 64 || lane < 32) && j < a.centroid_num;
        k[r] = ok ? cent_dist[j] : FLT_MAX;
        v[r] = ok ? j : kInvalid;
    }
    WaveNet<MAX_CENTROID>::sort(k, v, lane);
    wave_sync();
#pragma unroll
    for (int r = 0; r < NR; r++) {
        const uint32_t e = NR * lane + r;
        if ((MAX_CENTROID >= 64 || lane < 32) && e < a.centroid_num) {
            cent_dist[e] = k[r];
            cent_id[e] = v[r];
        }
    }
    wave_sync();
    uint32_t* out = a.segment_ids + static_cast<size_t>(q) * a.centroid_num;
    const float d0 = cent_dist[0];
    uint32_t allow_num = 0;
    for (uint32_t base = 0; base < a.centroid_num; base += 64) {
        const uint32_t i = base + lane;
        const bool allow = i < a.centroid_num && (cent_dist[i] / d0 <= a.boundary_factor);
        if (i < a.centroid_num) out[i] = allow ? cent_id[i] : kInvalid;
        allow_num += __popcll(ballot(allow));
    }
    if (allow_num < a.min_segment_num) {
        const uint32_t need = a.min_segment_num - allow_num;
        for (uint32_t i = lane; i < need && allow_num + i < a.centroid_num; i += 64) out[allow_num + i] = cent_id[allow_num + i];
    }
}

// Queries grouped by the partitions they selected: counts, then offsets, then the lists.  With them a partition's
// search launches one wavefront per query that wants it instead of one per query of the batch.
__global__ __launch_bounds__(256) void group_count_kernel(const uint32_t* segment_ids, uint32_t total, uint32_t centroid_num, uint32_t* counts) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const uint32_t s = segment_ids[i];
    if (s < centroid_num) atomicAdd(&counts[s], 1u);
}
__global__ __launch_bounds__(256) void group_scan_kernel(uint32_t* counts, uint32_t centroid_num, uint32_t* offsets, uint32_t* cursor) {
    if (threadIdx.x == 0) {
        uint32_t run = 0;
        for (uint32_t s = 0; s < centroid_num; s++) {
            offsets[s] = run;
            cursor[s] = run;
            run += counts[s];
        }
        offsets[centroid_num] = run;
    }
}
__global__ __launch_bounds__(256) void group_fill_kernel(const uint32_t* segment_ids, uint32_t total, uint32_t centroid_num, uint32_t* cursor,
                                                         uint32_t* lists, uint32_t* pair_segment, uint32_t* pair_index) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const uint32_t s = segment_ids[i];
    uint32_t pos = kInvalid;
    if (s < centroid_num) {
        pos = atomicAdd(&cursor[s], 1u);
        lists[pos] = i / centroid_num;
        if (pair_segment) pair_segment[pos] = s;
    }
    if (pair_index) pair_index[i] = pos;
}

// Per query: the heads its pairs left behind are merged in ascending partition order, the order in which the
// partition-by-partition search merges them (result_merge, search_kernel.cuh:609-651), so the result is the same.
template <int MAX_TOPK>
__device__ __forceinline__ void merge_pairs(const uint32_t* segment_ids, const uint32_t* pair_index, const float* pair_dists, const uint32_t* pair_ids,
                                            uint32_t centroid_num, uint32_t top_k, float* final_dists, uint32_t* final_ids, int lane) {
    constexpr int NR = WaveNet<MAX_TOPK>::NR;
    const bool live = MAX_TOPK >= 64 || lane < 32;
    float k[NR];
    uint32_t v[NR];
#pragma unroll
    for (int r = 0; r < NR; r++) {
        k[r] = FLT_MAX;
        v[r] = kInvalid;
    }
    uint32_t last = kInvalid;   // partition merged last; the first pass takes the smallest id
    for (;;) {
        uint32_t best = kInvalid, best_slot = 0;
        for (uint32_t i = lane; i < centroid_num; i += 64) {
            const uint32_t s = segment_ids[i];
            if (s != kInvalid && (last == kInvalid || s > last) && s < best) { best = s; best_slot = i; }
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            const uint32_t ob = __shfl_xor(best, off), os = __shfl_xor(best_slot, off);
            if (ob < best) { best = ob; best_slot = os; }
        }
        if (best == kInvalid) break;
        last = best;
        const uint32_t p = pair_index[best_slot];
        const float* bd = pair_dists + static_cast<size_t>(p) * top_k;
        const uint32_t* bi = pair_ids + static_cast<size_t>(p) * top_k;
#pragma unroll
        for (int r = 0; r < NR; r++) {
            const uint32_t e = NR * lane + r;
            const uint32_t kk = MAX_TOPK - 1 - e;
            if (live && kk < top_k) {
                const float rk = bd[kk];
                if (k[r] > rk) {
                    k[r] = rk;
                    v[r] = bi[kk];
                }
            }
        }
        WaveNet<MAX_TOPK>::merge(k, v, lane);
#pragma unroll
        for (int r = 0; r < NR; r++) {   // what the stored running result holds between two merges: top_k entries
            const uint32_t e = NR * lane + r;
            if (!(live && e < top_k)) { k[r] = FLT_MAX; v[r] = kInvalid; }
        }
    }
#pragma unroll
    for (int r = 0; r < NR; r++) {
        const uint32_t e = NR * lane + r;
        if (live && e < top_k) {
            final_dists[e] = k[r];
            final_ids[e] = v[r];
        }
    }
}

__global__ __launch_bounds__(64) void merge_pairs_kernel(const uint32_t* segment_ids, const uint32_t* pair_index, const float* pair_dists,
                                                         const uint32_t* pair_ids, uint32_t query_num, uint32_t centroid_num, uint32_t top_k,
                                                         uint32_t max_topk, float* final_dists, uint32_t* final_ids) {
    const uint32_t q = blockIdx.x;
    if (q >= query_num) return;
    const int lane = lane_id();
    const uint32_t* seg = segment_ids + static_cast<size_t>(q) * centroid_num;
    const uint32_t* idx = pair_index + static_cast<size_t>(q) * centroid_num;
    float* fd = final_dists + static_cast<size_t>(q) * top_k;
    uint32_t* fi = final_ids + static_cast<size_t>(q) * top_k;
    switch (max_topk) {
        case 32: merge_pairs<32>(seg, idx, pair_dists, pair_ids, centroid_num, top_k, fd, fi, lane); break;
        case 64: merge_pairs<64>(seg, idx, pair_dists, pair_ids, centroid_num, top_k, fd, fi, lane); break;
        default: merge_pairs<128>(seg, idx, pair_dists, pair_ids, centroid_num, top_k, fd, fi, lane); break;
    }
}

struct SubArgs {
    const float* data;          // the staged partition
    const uint32_t* graph;      // partition-local ids
    const uint32_t* map;        // local id -> original id
    const float* queries;
    const uint32_t* segment_ids;
    const uint32_t* query_list;   // nullable: the queries that selected this partition (then segment_ids is not read)
    // pair mode (nullable pair_segment): block p searches query query_list[p] in partition pair_segment[p]; data / graph /
    // map are then the arrays of all partitions, addressed through segment_starts, and the beam head goes to pair_dists / pair_ids
    const uint32_t* pair_segment;
    const uint32_t* segment_starts;
    const uint32_t* segment_start_points;
    float* pair_dists;
    uint32_t* pair_ids;
    uint32_t* final_ids;
    float* final_dists;
    unsigned long long* counters;
    uint32_t query_num, centroid_num, segment_id, start_point, top_k, max_topk, list_len;
    BeamParams p;
};

// result_merge (search_kernel.cuh:609-651): best top_k of (running result, this partition's beam head)
template <int MAX_TOPK, int MAX_BEAM>
__device__ __forceinline__ void merge_result(const float* beam_dist, const uint32_t* beam_id, const uint32_t* map, float* final_dists,
                                             uint32_t* final_ids, uint32_t top_k, int lane) {
    constexpr int NR = WaveNet<MAX_TOPK>::NR;
    const bool live = MAX_TOPK >= 64 || lane < 32;
    float k[NR];
    uint32_t v[NR];
#pragma unroll
    for (int r = 0; r < NR; r++) {
        const uint32_t e = NR * lane + r;
        k[r] = (live && e < top_k) ? final_dists[e] : FLT_MAX;
        v[r] = (live && e < top_k) ? final_ids[e] : kInvalid;
        const uint32_t kk = MAX_TOPK - 1 - e;
        if (live && kk < top_k) {
            const float rk = beam_dist[kk];
            if (k[r] > rk) {
                k[r] = rk;
                v[r] = map[beam_id[kk] & kClean];
            }
        }
    }
    WaveNet<MAX_TOPK>::merge(k, v, lane);
#pragma unroll
    for (int r = 0; r < NR; r++) {
        const uint32_t e = NR * lane + r;
        if (live && e < top_k) {
            final_dists[e] = k[r];
            final_ids[e] = v[r];
        }
    }
}

// search_on_sub_kernel (search_kernel.cuh:653-765)
template <int MAX_CAND, int MAX_BEAM, int DIMV, bool WHOLE = false>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(MAX_BEAM > 256 && DIMV <= 4 ? 4 : 1)))   // as search_kernel
void search_sub_kernel(SubArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    auto* lds = reinterpret_cast<BeamLds<MAX_CAND>*>(smem);
    float* head_dist = reinterpret_cast<float*>(smem + sizeof(BeamLds<MAX_CAND>));   // beam head staged for the merge (128 pairs)
    uint32_t* head_id = reinterpret_cast<uint32_t*>(head_dist + 128);
    uint32_t* hash = head_id + 128;
    uint32_t qid = blockIdx.x;
    const float* data = a.data;
    const uint32_t* graph = a.graph;
    const uint32_t* map = a.map;
    uint32_t start_point = a.start_point;
    if (a.pair_segment) {
        if (qid >= a.list_len) return;
        const uint32_t seg = a.pair_segment[qid];
        const size_t start = a.segment_starts[seg];
        data += start * a.p.dim;
        graph += start * a.p.degree;
        map += start;
        start_point = a.segment_start_points[seg];
        if (start_point == kInvalid) {   // an empty partition: nothing to find
            for (uint32_t e = lane_id(); e < a.top_k; e += 64) {
                a.pair_dists[static_cast<size_t>(blockIdx.x) * a.top_k + e] = FLT_MAX;
                a.pair_ids[static_cast<size_t>(blockIdx.x) * a.top_k + e] = kInvalid;
            }
            return;
        }
        qid = a.query_list[qid];
    } else if (a.query_list) {
        if (qid >= a.list_len) return;
        qid = a.query_list[qid];
    } else {
        if (qid >= a.query_num) return;
        bool is_search = false;   // wave-uniform scan of this query's partition list
        for (uint32_t i = 0; i < a.centroid_num; i++) {
            const uint32_t s = a.segment_ids[static_cast<size_t>(qid) * a.centroid_num + i];
            if (s == a.segment_id) { is_search = true; break; }
            if (s == kInvalid) break;
        }
        if (!is_search) return;
    }

    Beam<MAX_CAND, MAX_BEAM, DIMV, false, WHOLE> b;
    b.init(lds, hash, a.p, a.queries + static_cast<size_t>(qid) * a.p.dim);
    b.expand(start_point, graph, data, kInvalid, kInvalid);   // get_init with point_id = 0xffffffff
    b.run(graph, data, kInvalid);

    constexpr int NB = MAX_BEAM / 64;
    if (a.pair_segment) {   // the head of this pair's beam, ids already as input row numbers; merged per query afterwards
#pragma unroll
        for (int r = 0; r < NB; r++) {
            const uint32_t e = NB * b.lane + r;
            if (e < a.top_k) {
                const float d = b.bk[r];
                a.pair_dists[static_cast<size_t>(blockIdx.x) * a.top_k + e] = d;
                a.pair_ids[static_cast<size_t>(blockIdx.x) * a.top_k + e] = d < FLT_MAX ? map[b.bv[r] & kClean] : kInvalid;
            }
        }
        b.flush_counters(a.counters);
        return;
    }
#pragma unroll
    for (int r = 0; r < NB; r++) {
        const uint32_t e = NB * b.lane + r;
        if (e < 128) {
            head_dist[e] = b.bk[r];
            head_id[e] = b.bv[r];
        }
    }
    wave_sync();
    float* fd = a.final_dists + static_cast<size_t>(qid) * a.top_k;
    uint32_t* fi = a.final_ids + static_cast<size_t>(qid) * a.top_k;
    switch (a.max_topk) {   // kernel_config.cuh:312-323
        case 32: merge_result<32, MAX_BEAM>(head_dist, head_id, map, fd, fi, a.top_k, b.lane); break;
        case 64: merge_result<64, MAX_BEAM>(head_dist, head_id, map, fd, fi, a.top_k, b.lane); break;
        default: merge_result<128, MAX_BEAM>(head_dist, head_id, map, fd, fi, a.top_k, b.lane); break;
    }
    b.flush_counters(a.counters);
}

using sub_fn = void (*)(SubArgs);

template <int MAX_CAND, int MAX_BEAM, bool WHOLE = false>
sub_fn pick_sub_dim(uint32_t dim) {
    if (dim <= 128) return search_sub_kernel<MAX_CAND, MAX_BEAM, 1, WHOLE>;
    if (dim <= 256) return search_sub_kernel<MAX_CAND, MAX_BEAM, 2, WHOLE>;
    if (dim <= 512) return search_sub_kernel<MAX_CAND, MAX_BEAM, 4, WHOLE>;
    if (dim <= 1024) return search_sub_kernel<MAX_CAND, MAX_BEAM, 8, WHOLE>;
    if (dim <= 2048) return search_sub_kernel<MAX_CAND, MAX_BEAM, 16, WHOLE>;
    return search_sub_kernel<MAX_CAND, MAX_BEAM, 32, WHOLE>;
}
template <int MAX_CAND>
sub_fn pick_sub_beam(uint32_t beam, uint32_t dim) {
    if (beam <= 64) return pick_sub_dim<MAX_CAND, 64>(dim);
    if (beam <= 128) return pick_sub_dim<MAX_CAND, 128>(dim);
    if (beam <= 256) return pick_sub_dim<MAX_CAND, 256>(dim);
    if (beam == 512) return pick_sub_dim<MAX_CAND, 512, true>(dim);   // the whole of the widest beam: merged in the registers
    return pick_sub_dim<MAX_CAND, 512>(dim);
}

}  // namespace glide

using namespace glide;

extern "C" int glide_hip_select_segments(const float* queries, uint32_t query_num, uint32_t dim, const float* centroids, uint32_t centroid_num,
                                         uint32_t min_segment_num, float boundary_factor, int metric, uint32_t* segment_ids, void* stream) {
    if (!queries || !centroids || !segment_ids || dim == 0 || centroid_num == 0) return GLIDE_ERR_BAD_ARGUMENT;
    if (metric != GLIDE_METRIC_EUCLIDEAN && metric != GLIDE_METRIC_COSINE) return GLIDE_ERR_BAD_ARGUMENT;
    if (centroid_num > 256 || dim % 4 != 0) return GLIDE_ERR_UNSUPPORTED;   // kernel_config.cuh:290-304
    if (query_num == 0) return GLIDE_OK;
    SelectArgs a{queries, centroids, segment_ids, query_num, dim, centroid_num, min_segment_num, boundary_factor, metric};
    const size_t lds = round_up32(centroid_num) * 8;
    hipStream_t s = as_stream(stream);
    if (centroid_num <= 32) hipLaunchKernelGGL(select_segments_kernel<32>, dim3(query_num), dim3(64), lds, s, a);
    else if (centroid_num <= 64) hipLaunchKernelGGL(select_segments_kernel<64>, dim3(query_num), dim3(64), lds, s, a);
    else if (centroid_num <= 128) hipLaunchKernelGGL(select_segments_kernel<128>, dim3(query_num), dim3(64), lds, s, a);
    else hipLaunchKernelGGL(select_segments_kernel<256>, dim3(query_num), dim3(64), lds, s, a);
    return launch_status();
}

namespace {
int launch_search_sub(const float* segment_data, uint32_t dim, const uint32_t* segment_graph, uint32_t graph_degree, const uint32_t* segment_map,
                      const float* queries, uint32_t query_num, const uint32_t* segment_ids, const uint32_t* query_list, uint32_t list_len,
                      uint32_t centroid_num, uint32_t segment_id, uint32_t start_point, uint32_t top_k, uint32_t beam, uint32_t max_iterations,
                      uint32_t min_iterations, uint32_t hash_bit, uint32_t hash_reset_interval, int metric, uint32_t* final_ids,
                      float* final_dists, unsigned long long* counters, void* stream) {
    if (!segment_data || !segment_graph || !segment_map || !queries || (!segment_ids && !query_list) || !final_ids || !final_dists)
        return GLIDE_ERR_BAD_ARGUMENT;
    if (dim == 0 || graph_degree == 0 || centroid_num == 0 || beam == 0 || top_k == 0 || max_iterations == 0) return GLIDE_ERR_BAD_ARGUMENT;
    if (metric != GLIDE_METRIC_EUCLIDEAN && metric != GLIDE_METRIC_COSINE) return GLIDE_ERR_BAD_ARGUMENT;
    if (query_num == 0 || (query_list && list_len == 0)) return GLIDE_OK;
    if (graph_degree > 256 || !beam_supported(beam) || dim % 4 != 0 || dim > 4096 || top_k > beam || top_k > 128 || hash_bit < 1 || hash_bit > 13)
        return GLIDE_ERR_UNSUPPORTED;   // top_k buckets: kernel_config.cuh:312-323
    SubArgs a;
    a.data = segment_data;
    a.graph = segment_graph;
    a.map = segment_map;
    a.queries = queries;
    a.segment_ids = segment_ids;
    a.query_list = query_list;
    a.list_len = list_len;
    a.pair_segment = nullptr;
    a.segment_starts = nullptr;
    a.segment_start_points = nullptr;
    a.pair_dists = nullptr;
    a.pair_ids = nullptr;
    a.final_ids = final_ids;
    a.final_dists = final_dists;
    a.counters = counters;
    a.query_num = query_num;
    a.centroid_num = centroid_num;
    a.segment_id = segment_id;
    a.start_point = start_point;
    a.top_k = top_k;
    a.max_topk = top_k <= 32 ? 32 : (top_k <= 64 ? 64 : 128);
    a.p = BeamParams{beam, graph_degree, dim, hash_bit, hash_reset_interval ? hash_reset_interval : 1, max_iterations, min_iterations, metric};
    sub_fn fn = graph_degree <= 64 ? pick_sub_beam<64>(beam, dim) : graph_degree <= 128 ? pick_sub_beam<128>(beam, dim) : pick_sub_beam<256>(beam, dim);
    const size_t lds_bytes = beam_lds_bytes(graph_degree) + 128 * 8 + (size_t{1} << hash_bit) * sizeof(uint32_t);
    GLIDE_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
    hipLaunchKernelGGL(fn, dim3(query_list ? list_len : query_num), dim3(64), lds_bytes, as_stream(stream), a);
    return launch_status();
}
}  // namespace

extern "C" int glide_hip_search_sub(const float* segment_data, uint32_t dim, const uint32_t* segment_graph, uint32_t graph_degree,
                                    const uint32_t* segment_map, const float* queries, uint32_t query_num, const uint32_t* segment_ids,
                                    uint32_t centroid_num, uint32_t segment_id, uint32_t start_point, uint32_t top_k, uint32_t beam,
                                    uint32_t max_iterations, uint32_t min_iterations, uint32_t hash_bit, uint32_t hash_reset_interval,
                                    int metric, uint32_t* final_ids, float* final_dists, unsigned long long* counters, void* stream) {
    if (!segment_ids) return GLIDE_ERR_BAD_ARGUMENT;
    return launch_search_sub(segment_data, dim, segment_graph, graph_degree, segment_map, queries, query_num, segment_ids, nullptr, 0, centroid_num,
                             segment_id, start_point, top_k, beam, max_iterations, min_iterations, hash_bit, hash_reset_interval, metric, final_ids,
                             final_dists, counters, stream);
}

extern "C" int glide_hip_search_sub_listed(const float* segment_data, uint32_t dim, const uint32_t* segment_graph, uint32_t graph_degree,
                                           const uint32_t* segment_map, const float* queries, uint32_t query_num, const uint32_t* query_list,
                                           uint32_t list_len, uint32_t segment_id, uint32_t start_point, uint32_t top_k, uint32_t beam,
                                           uint32_t max_iterations, uint32_t min_iterations, uint32_t hash_bit, uint32_t hash_reset_interval,
                                           int metric, uint32_t* final_ids, float* final_dists, unsigned long long* counters, void* stream) {
    if (!query_list && list_len) return GLIDE_ERR_BAD_ARGUMENT;
    if (list_len == 0) return GLIDE_OK;
    return launch_search_sub(segment_data, dim, segment_graph, graph_degree, segment_map, queries, query_num, nullptr, query_list, list_len, 1,
                             segment_id, start_point, top_k, beam, max_iterations, min_iterations, hash_bit, hash_reset_interval, metric, final_ids,
                             final_dists, counters, stream);
}

extern "C" size_t glide_hip_group_queries_workspace_bytes(uint32_t centroid_num) { return (static_cast<size_t>(centroid_num) + 1) * 4 + 256; }

extern "C" int glide_hip_group_queries(const uint32_t* segment_ids, uint32_t query_num, uint32_t centroid_num, uint32_t* counts, uint32_t* offsets,
                                       uint32_t* lists, void* workspace, size_t workspace_bytes, void* stream) {
    if (!segment_ids || !counts || !offsets || !lists || !workspace || centroid_num == 0) return GLIDE_ERR_BAD_ARGUMENT;
    if (workspace_bytes < glide_hip_group_queries_workspace_bytes(centroid_num)) return GLIDE_ERR_BAD_ARGUMENT;
    if (static_cast<unsigned long long>(query_num) * centroid_num >= 0xffffffffull) return GLIDE_ERR_UNSUPPORTED;
    hipStream_t s = as_stream(stream);
    int rc = glide_hip_fill_u32(counts, 0u, centroid_num, stream);
    if (rc != GLIDE_OK) return rc;
    const uint32_t total = query_num * centroid_num;
    uint32_t* cursor = static_cast<uint32_t*>(workspace);
    if (total) hipLaunchKernelGGL(group_count_kernel, dim3(ceil_div(total, 256)), dim3(256), 0, s, segment_ids, total, centroid_num, counts);
    hipLaunchKernelGGL(group_scan_kernel, dim3(1), dim3(256), 0, s, counts, centroid_num, offsets, cursor);
    if (total) hipLaunchKernelGGL(group_fill_kernel, dim3(ceil_div(total, 256)), dim3(256), 0, s, segment_ids, total, centroid_num, cursor, lists,
                                  static_cast<uint32_t*>(nullptr), static_cast<uint32_t*>(nullptr));
    return launch_status();
}

namespace {
size_t align256(size_t x) { return (x + 255) / 256 * 256; }
struct PartitionSearchLayout { size_t counts, offsets, cursor, lists, pair_segment, pair_index, pair_dists, pair_ids, total; };
PartitionSearchLayout partition_search_layout(uint32_t query_num, uint32_t centroid_num, uint32_t top_k) {
    PartitionSearchLayout l;
    const size_t pairs = static_cast<size_t>(query_num) * centroid_num;   // every query could select every partition
    size_t off = 0;
    auto take = [&off](size_t bytes) { size_t o = off; off += align256(bytes); return o; };
    l.counts = take(static_cast<size_t>(centroid_num) * 4);
    l.offsets = take((static_cast<size_t>(centroid_num) + 1) * 4);
    l.cursor = take(static_cast<size_t>(centroid_num) * 4);
    l.lists = take(pairs * 4);
    l.pair_segment = take(pairs * 4);
    l.pair_index = take(pairs * 4);
    l.pair_dists = take(pairs * top_k * 4);
    l.pair_ids = take(pairs * top_k * 4);
    l.total = off;
    return l;
}
}  // namespace

extern "C" size_t glide_hip_search_partitions_workspace_bytes(uint32_t query_num, uint32_t centroid_num, uint32_t top_k) {
    return partition_search_layout(query_num, centroid_num, top_k).total;
}

extern "C" int glide_hip_search_partitions(const float* data, uint32_t dim, const uint32_t* graph, uint32_t graph_degree, const uint32_t* map,
                                           const uint32_t* segment_starts, const uint32_t* segment_start_points, uint32_t segment_num,
                                           const float* queries, uint32_t query_num, const uint32_t* segment_ids, uint32_t top_k, uint32_t beam,
                                           uint32_t max_iterations, uint32_t min_iterations, uint32_t hash_bit, uint32_t hash_reset_interval,
                                           int metric, uint32_t* final_ids, float* final_dists, void* workspace, size_t workspace_bytes,
                                           unsigned long long* counters, void* stream) {
    if (!data || !graph || !map || !segment_starts || !segment_start_points || !queries || !segment_ids || !final_ids || !final_dists || !workspace)
        return GLIDE_ERR_BAD_ARGUMENT;
    if (dim == 0 || graph_degree == 0 || segment_num == 0 || beam == 0 || top_k == 0 || max_iterations == 0) return GLIDE_ERR_BAD_ARGUMENT;
    if (metric != GLIDE_METRIC_EUCLIDEAN && metric != GLIDE_METRIC_COSINE) return GLIDE_ERR_BAD_ARGUMENT;
    if (query_num == 0) return GLIDE_OK;
    if (graph_degree > 256 || !beam_supported(beam) || dim % 4 != 0 || dim > 4096 || top_k > beam || top_k > 128 || hash_bit < 1 || hash_bit > 13)
        return GLIDE_ERR_UNSUPPORTED;
    if (static_cast<unsigned long long>(query_num) * segment_num >= 0xffffffffull) return GLIDE_ERR_UNSUPPORTED;   // pairs are numbered with 32 bits
    const PartitionSearchLayout l = partition_search_layout(query_num, segment_num, top_k);
    if (workspace_bytes < l.total || reinterpret_cast<uintptr_t>(workspace) % 8) return GLIDE_ERR_BAD_ARGUMENT;
    hipStream_t s = as_stream(stream);
    unsigned char* w = static_cast<unsigned char*>(workspace);
    uint32_t* counts = reinterpret_cast<uint32_t*>(w + l.counts);
    uint32_t* offsets = reinterpret_cast<uint32_t*>(w + l.offsets);
    uint32_t* cursor = reinterpret_cast<uint32_t*>(w + l.cursor);
    uint32_t* lists = reinterpret_cast<uint32_t*>(w + l.lists);
    uint32_t* pair_segment = reinterpret_cast<uint32_t*>(w + l.pair_segment);
    uint32_t* pair_index = reinterpret_cast<uint32_t*>(w + l.pair_index);
    float* pair_dists = reinterpret_cast<float*>(w + l.pair_dists);
    uint32_t* pair_ids = reinterpret_cast<uint32_t*>(w + l.pair_ids);
    int rc = glide_hip_fill_u32(counts, 0u, segment_num, stream);
    if (rc != GLIDE_OK) return rc;
    const uint32_t total = query_num * segment_num;
    hipLaunchKernelGGL(group_count_kernel, dim3(ceil_div(total, 256)), dim3(256), 0, s, segment_ids, total, segment_num, counts);
    hipLaunchKernelGGL(group_scan_kernel, dim3(1), dim3(256), 0, s, counts, segment_num, offsets, cursor);
    hipLaunchKernelGGL(group_fill_kernel, dim3(ceil_div(total, 256)), dim3(256), 0, s, segment_ids, total, segment_num, cursor, lists, pair_segment,
                       pair_index);
    uint32_t pairs = 0;   // the grid of the search: one wavefront per (query, selected partition)
    GLIDE_HIP_TRY(hipMemcpyAsync(&pairs, offsets + segment_num, sizeof(uint32_t), hipMemcpyDeviceToHost, s));
    GLIDE_HIP_TRY(hipStreamSynchronize(s));
    if (pairs) {
        SubArgs a;
        a.data = data;
        a.graph = graph;
        a.map = map;
        a.queries = queries;
        a.segment_ids = nullptr;
        a.query_list = lists;
        a.pair_segment = pair_segment;
        a.segment_starts = segment_starts;
        a.segment_start_points = segment_start_points;
        a.pair_dists = pair_dists;
        a.pair_ids = pair_ids;
        a.final_ids = nullptr;
        a.final_dists = nullptr;
        a.counters = counters;
        a.query_num = query_num;
        a.centroid_num = segment_num;
        a.segment_id = 0;
        a.start_point = 0;
        a.top_k = top_k;
        a.max_topk = top_k <= 32 ? 32 : (top_k <= 64 ? 64 : 128);
        a.list_len = pairs;
        a.p = BeamParams{beam, graph_degree, dim, hash_bit, hash_reset_interval ? hash_reset_interval : 1, max_iterations, min_iterations, metric};
        sub_fn fn = graph_degree <= 64 ? pick_sub_beam<64>(beam, dim) : graph_degree <= 128 ? pick_sub_beam<128>(beam, dim) : pick_sub_beam<256>(beam, dim);
        const size_t lds_bytes = beam_lds_bytes(graph_degree) + 128 * 8 + (size_t{1} << hash_bit) * sizeof(uint32_t);
        GLIDE_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
        hipLaunchKernelGGL(fn, dim3(pairs), dim3(64), lds_bytes, s, a);
    }
    hipLaunchKernelGGL(merge_pairs_kernel, dim3(query_num), dim3(64), 0, s, segment_ids, pair_index, pair_dists, pair_ids, query_num, segment_num, top_k,
                       top_k <= 32 ? 32u : (top_k <= 64 ? 64u : 128u), final_dists, final_ids);
    return launch_status();
}
