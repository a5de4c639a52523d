// glide_hip_search: one query per wavefront beam search over the finished index.
// Reference: search_kernel (search_kernel.cuh:393-490) launched by GLIDE::search (glide_impl.cuh:370-454).
#include "beam.hpp"
#include "host_util.hpp"

namespace glide {

struct SearchArgs {
    const float* data;
    const uint32_t* graph;
    const float* centroids;
    const uint32_t* start_points;
    const float* queries;
    uint32_t* result_ids;
    float* result_dists;
    unsigned long long* counters;
    uint32_t centroid_num, max_centroid, top_k, query_num;
    BeamParams p;
};

template <int DIMV, bool TEAM = false>
__device__ __forceinline__ uint32_t pick_centroid(uint32_t max_centroid, const RowRegs<DIMV>& q, const float* centroids,
                                                  uint32_t centroid_num, uint32_t dim, int metric, float* scratch, int lane) {
    switch (max_centroid) {  // bucket chosen like reference kernel_config.cuh:161-171
        case 32: return nearest_centroid<32, DIMV, TEAM>(q, centroids, centroid_num, dim, metric, scratch, lane);
        case 64: return nearest_centroid<64, DIMV, TEAM>(q, centroids, centroid_num, dim, metric, scratch, lane);
        case 128: return nearest_centroid<128, DIMV, TEAM>(q, centroids, centroid_num, dim, metric, scratch, lane);
        default: return nearest_centroid<256, DIMV, TEAM>(q, centroids, centroid_num, dim, metric, scratch, lane);
    }
}

template <int MAX_CAND, int MAX_BEAM, int DIMV, bool WHOLE = false>
__device__ __forceinline__ void search_body(const SearchArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    auto* lds = reinterpret_cast<BeamLds<MAX_CAND>*>(smem);
    float* cent = reinterpret_cast<float*>(smem + sizeof(BeamLds<MAX_CAND>));
    uint32_t* hash = reinterpret_cast<uint32_t*>(cent + round_up32(a.centroid_num));
    // a wavefront takes queries blockIdx.x, blockIdx.x + gridDim.x, ... (the host sizes the grid)
    for (uint32_t qid = blockIdx.x; qid < a.query_num; qid += gridDim.x) {
        Beam<MAX_CAND, MAX_BEAM, DIMV, false, WHOLE> b;
        b.init(lds, hash, a.p, a.queries + static_cast<size_t>(qid) * a.p.dim);
        const uint32_t c0 = pick_centroid<DIMV>(a.max_centroid, b.q, a.centroids, a.centroid_num, a.p.dim, a.p.metric, cent, b.lane);
        const uint32_t entry = a.start_points[c0];
        b.expand(entry, a.graph, a.data, kInvalid, kInvalid);  // result_init: entry node itself is never scored
        b.run(a.graph, a.data, kInvalid);

        constexpr int NB = MAX_BEAM / 64;
#pragma unroll
        for (int r = 0; r < NB; r++) {
            const uint32_t e = NB * b.lane + r;
            if (e < a.top_k) {
                a.result_ids[static_cast<size_t>(qid) * a.top_k + e] = b.bv[r] & kClean;
                a.result_dists[static_cast<size_t>(qid) * a.top_k + e] = b.bk[r];
            }
        }
        b.flush_counters(a.counters);
        wave_sync();   // the next query reuses the LDS
    }
}

template <int MAX_CAND, int MAX_BEAM, int DIMV, bool WHOLE = false>
__global__ __launch_bounds__(64) void search_kernel(SearchArgs a) {
    search_body<MAX_CAND, MAX_BEAM, DIMV, WHOLE>(a);
}
// The beam-256 kernels are bound by the vector ALU (sorting networks) and need 103 registers, one wavefront per SIMD
// short of the next occupancy step: held to five wavefronts per SIMD (96 registers, five of them spilled) they run
// 5 % faster.  Other beams are either already there or would spill much more.
template <int MAX_CAND, int MAX_BEAM, int DIMV>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(5, 5))) void search_kernel_dense(SearchArgs a) {
    search_body<MAX_CAND, MAX_BEAM, DIMV>(a);
}

// Small batches of long rows (more than 256 dims): a team of kTeam wavefronts per query.  Wavefront 0 owns the search
// (beam, visited set, sorting networks) exactly as in search_kernel; between two of its passes every wavefront of the
// team scores a share of the expansion's candidate rows.  One wavefront can keep only a few 2-4 KB rows in flight in its
// registers, and a search is a chain of dependent expansions: while the batch leaves SIMDs idle, a team gives a query
// kTeam times the bytes on their way and an expansion takes one or two memory round trips instead of six (64 queries of
// 960 dims: 1.9 times the throughput at beams up to 256, 1.3 times above).  Once a batch fills the chip on its own
// (about two wavefronts per SIMD) the row gathers run at the rate the memory system sustains for scattered rows either
// way and the team only adds its barriers, so larger batches keep one wavefront per query.  The query row sits in LDS
// once per team (RefInLds) so that the registers hold rows in flight; every distance is summed in the order
// search_kernel sums it, so results are identical.
constexpr int kTeam = 4;

template <int DIMV>
struct TeamShape {
    static constexpr int U = DIMV >= 16 ? 1 : (DIMV == 8 ? 2 : 4);   // row steps in flight per wavefront: 64 row registers either way
    static constexpr size_t query_bytes = sizeof(float4) * RowShape<DIMV>::NV * RowShape<DIMV>::LPR;
};

template <int MAX_CAND, int MAX_BEAM, int DIMV, bool WHOLE = false>
__global__ __launch_bounds__(64 * kTeam) void search_team_kernel(SearchArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    using Shape = RowShape<DIMV>;
    auto* lds = reinterpret_cast<BeamLds<MAX_CAND>*>(smem);
    float* cent = reinterpret_cast<float*>(smem + sizeof(BeamLds<MAX_CAND>));
    float4* qlds = reinterpret_cast<float4*>(cent + round_up32(a.centroid_num));
    uint32_t* ctl = reinterpret_cast<uint32_t*>(qlds + Shape::NV * Shape::LPR);   // [0] rows to score, [1] search over
    uint32_t* hash = ctl + 4;
    const uint32_t wave = threadIdx.x >> 6;
    const int lane = lane_id();
    for (uint32_t qid = blockIdx.x; qid < a.query_num; qid += gridDim.x) {
        Beam<MAX_CAND, MAX_BEAM, DIMV, true, WHOLE> b;
        uint32_t iter = 0;
        bool terminate = false;
        if (wave == 0) {
            b.init(lds, hash, a.p, a.queries + static_cast<size_t>(qid) * a.p.dim);
            if (Shape::row_of_lane(lane) == 0) {
#pragma unroll
                for (int c = 0; c < Shape::NV; c++) qlds[c * Shape::LPR + Shape::lane_in_row(lane)] = b.q.v[c];
            }
            const uint32_t c0 = pick_centroid<DIMV, true>(a.max_centroid, b.q, a.centroids, a.centroid_num, a.p.dim, a.p.metric, cent, lane);
            const uint32_t nv = b.expand_list(a.start_points[c0], a.graph, kInvalid, kInvalid);   // result_init: the entry node itself is never scored
            if (lane == 0) {
                ctl[0] = nv;
                ctl[1] = 0;
            }
        }
        __syncthreads();
        while (true) {
            const uint32_t nv = ctl[0];
            score_share<DIMV, TeamShape<DIMV>::U>(RefInLds<DIMV>{qlds}, a.data, a.p.dim, a.p.metric, 0, nv, lane, wave, kTeam,
                                                  [lds](uint32_t idx) { return lds->cand_id[lds->vlist[idx]]; },
                                                  [lds](uint32_t idx, float d) { lds->cand_dist[lds->vlist[idx]] = d; });
            __syncthreads();
            if (wave == 0) {
                uint32_t next = 0;
                const bool more = b.step_to_list(iter, terminate, a.graph, kInvalid, next);
                if (lane == 0) {
                    ctl[0] = next;
                    ctl[1] = more ? 0u : 1u;
                }
            }
            __syncthreads();
            if (ctl[1] != 0) break;
        }
        if (wave == 0) {
            constexpr int NB = MAX_BEAM / 64;
#pragma unroll
            for (int r = 0; r < NB; r++) {
                const uint32_t e = NB * lane + r;
                if (e < a.top_k) {
                    a.result_ids[static_cast<size_t>(qid) * a.top_k + e] = b.bv[r] & kClean;
                    a.result_dists[static_cast<size_t>(qid) * a.top_k + e] = b.bk[r];
                }
            }
            b.flush_counters(a.counters);
        }
        __syncthreads();   // the next query reuses the LDS
    }
}

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
__global__ __launch_bounds__(64) void search_sub_kernel(SubArgs a) {
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

using search_fn = void (*)(SearchArgs);
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

template <int MAX_CAND, int MAX_BEAM, bool WHOLE = false>
search_fn pick_dim(uint32_t dim) {
    if constexpr (MAX_BEAM == 256 && MAX_CAND <= 128) {
        if (dim <= 128) return search_kernel_dense<MAX_CAND, MAX_BEAM, 1>;
        if (dim <= 256) return search_kernel_dense<MAX_CAND, MAX_BEAM, 2>;
        if (dim <= 512) return search_kernel_dense<MAX_CAND, MAX_BEAM, 4>;
    }
    if (dim <= 128) return search_kernel<MAX_CAND, MAX_BEAM, 1, WHOLE>;
    if (dim <= 256) return search_kernel<MAX_CAND, MAX_BEAM, 2, WHOLE>;
    if (dim <= 512) return search_kernel<MAX_CAND, MAX_BEAM, 4, WHOLE>;
    if (dim <= 1024) return search_kernel<MAX_CAND, MAX_BEAM, 8, WHOLE>;
    if (dim <= 2048) return search_kernel<MAX_CAND, MAX_BEAM, 16, WHOLE>;
    return search_kernel<MAX_CAND, MAX_BEAM, 32, WHOLE>;
}
template <int MAX_CAND, int MAX_BEAM, bool WHOLE = false>
search_fn pick_team_dim(uint32_t dim) {
    if (dim <= 512) return search_team_kernel<MAX_CAND, MAX_BEAM, 4, WHOLE>;
    if (dim <= 1024) return search_team_kernel<MAX_CAND, MAX_BEAM, 8, WHOLE>;
    if (dim <= 2048) return search_team_kernel<MAX_CAND, MAX_BEAM, 16, WHOLE>;
    return search_team_kernel<MAX_CAND, MAX_BEAM, 32, WHOLE>;
}
template <int MAX_CAND>
search_fn pick_team_beam(uint32_t beam, uint32_t dim) {
    if (beam <= 64) return pick_team_dim<MAX_CAND, 64>(dim);
    if (beam <= 128) return pick_team_dim<MAX_CAND, 128>(dim);
    if (beam <= 256) return pick_team_dim<MAX_CAND, 256>(dim);
    if (beam == 512) return pick_team_dim<MAX_CAND, 512, true>(dim);
    return pick_team_dim<MAX_CAND, 512>(dim);
}
template <int MAX_CAND>
search_fn pick_beam(uint32_t beam, uint32_t dim) {
    if (beam <= 64) return pick_dim<MAX_CAND, 64>(dim);
    if (beam <= 128) return pick_dim<MAX_CAND, 128>(dim);
    if (beam <= 256) return pick_dim<MAX_CAND, 256>(dim);
    if (beam == 512) return pick_dim<MAX_CAND, 512, true>(dim);
    return pick_dim<MAX_CAND, 512>(dim);
}

// Grid size for the one-query-per-wavefront search kernel.  With small beams the kernel is bound by row gathers; when
// the batch is a little larger than what the chip holds at once (10 000 queries against 8 192 wavefront slots),
// hardware dispatch runs one full round and a thin, latency-bound tail.  Equal rounds are faster: the grid is the
// batch divided by the number of rounds and every wavefront loops over its share.  Larger beams are bound by the
// sorting networks and keep one workgroup per query.
size_t simd_count() {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) return 0;
    return static_cast<size_t>(cus) * 4;
}

uint32_t balanced_grid(uint32_t items, uint32_t beam, size_t lds_bytes) {
    if (beam > 64) return items;
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
        return items;
    const size_t by_lds = lds_bytes ? (160 * 1024) / lds_bytes : 32;
    const size_t slots = static_cast<size_t>(cus) * (by_lds < 32 ? by_lds : 32);   // 4 SIMDs x 8 wavefronts per CU
    if (slots == 0 || items <= slots) return items;
    const size_t rounds = (items + slots - 1) / slots;
    return static_cast<uint32_t>((items + rounds - 1) / rounds);
}

}  // namespace glide

using namespace glide;

namespace {
int launch_search(const float* data, uint32_t num, uint32_t dim, const uint32_t* graph, uint32_t graph_degree, const float* centroids,
                  uint32_t centroid_num, bool rank_all_centroids, const uint32_t* start_points, const float* queries, uint32_t query_num,
                  uint32_t top_k, uint32_t beam, uint32_t max_iterations, uint32_t min_iterations, uint32_t hash_bit,
                  uint32_t hash_reset_interval, int metric, uint32_t* result_ids, float* result_dists, unsigned long long* counters,
                  void* stream) {
    if (!data || !graph || !centroids || !start_points || !queries || !result_ids || !result_dists) return GLIDE_ERR_BAD_ARGUMENT;
    if (num == 0 || dim == 0 || graph_degree == 0 || centroid_num == 0 || beam == 0 || top_k == 0 || max_iterations == 0)
        return GLIDE_ERR_BAD_ARGUMENT;
    if (metric != GLIDE_METRIC_EUCLIDEAN && metric != GLIDE_METRIC_COSINE) return GLIDE_ERR_BAD_ARGUMENT;
    if (query_num == 0) return GLIDE_OK;
    if (graph_degree > 256 || beam > 512 || centroid_num > 256 || dim % 4 != 0 || dim > 4096 || top_k > beam ||
        hash_bit < 1 || hash_bit > 13)
        return GLIDE_ERR_UNSUPPORTED;
    if (reinterpret_cast<uintptr_t>(data) % 16 || reinterpret_cast<uintptr_t>(queries) % 16 ||
        reinterpret_cast<uintptr_t>(centroids) % 16)
        return GLIDE_ERR_BAD_ARGUMENT;

    SearchArgs a;
    a.data = data;
    a.graph = graph;
    a.centroids = centroids;
    a.start_points = start_points;
    a.queries = queries;
    a.result_ids = result_ids;
    a.result_dists = result_dists;
    a.counters = counters;
    a.centroid_num = centroid_num;
    // reference kernel_config.cuh:161-171: bucket from graph_degree once there are more than 32 centroids
    a.max_centroid = centroid_num <= 32 ? 32 : (graph_degree <= 64 ? 64 : (graph_degree <= 128 ? 128 : 256));
    if (rank_all_centroids) a.max_centroid = centroid_num <= 32 ? 32 : (centroid_num <= 64 ? 64 : (centroid_num <= 128 ? 128 : 256));
    a.top_k = top_k;
    a.query_num = query_num;
    a.p.beam = beam;
    a.p.degree = graph_degree;
    a.p.dim = dim;
    a.p.hash_bit = hash_bit;
    a.p.reset_interval = hash_reset_interval ? hash_reset_interval : 1;
    a.p.max_iterations = max_iterations;
    a.p.min_iterations = min_iterations;
    a.p.metric = metric;

    const bool team = dim > 256 && static_cast<size_t>(query_num) * kTeam <= 2 * simd_count();   // see search_team_kernel
    search_fn fn;
    if (team) fn = graph_degree <= 64 ? pick_team_beam<64>(beam, dim) : graph_degree <= 128 ? pick_team_beam<128>(beam, dim) : pick_team_beam<256>(beam, dim);
    else fn = graph_degree <= 64 ? pick_beam<64>(beam, dim) : graph_degree <= 128 ? pick_beam<128>(beam, dim) : pick_beam<256>(beam, dim);
    const size_t lds_bytes = beam_lds_bytes(graph_degree) + round_up32(centroid_num) * sizeof(float) +
                             (size_t{1} << hash_bit) * sizeof(uint32_t) + beam_stage_bytes(beam, beam == 512) +
                             (team ? (dim <= 512 ? TeamShape<4>::query_bytes : dim <= 1024 ? TeamShape<8>::query_bytes : dim <= 2048 ? TeamShape<16>::query_bytes : TeamShape<32>::query_bytes) + 16 : 0);
    GLIDE_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
    if (team) hipLaunchKernelGGL(fn, dim3(query_num), dim3(64 * kTeam), lds_bytes, as_stream(stream), a);
    else hipLaunchKernelGGL(fn, dim3(balanced_grid(query_num, beam, lds_bytes)), dim3(64), lds_bytes, as_stream(stream), a);
    return launch_status();
}
}  // namespace

extern "C" int glide_hip_search(const float* data, uint32_t num, uint32_t dim, const uint32_t* graph, uint32_t graph_degree,
                                const float* centroids, uint32_t centroid_num, const uint32_t* start_points,
                                const float* queries, uint32_t query_num, uint32_t top_k, uint32_t beam,
                                uint32_t max_iterations, uint32_t min_iterations, uint32_t hash_bit,
                                uint32_t hash_reset_interval, int metric, uint32_t* result_ids, float* result_dists,
                                unsigned long long* counters, void* stream) {
    return launch_search(data, num, dim, graph, graph_degree, centroids, centroid_num, false, start_points, queries, query_num, top_k, beam,
                         max_iterations, min_iterations, hash_bit, hash_reset_interval, metric, result_ids, result_dists, counters, stream);
}

extern "C" int glide_hip_search_merged(const float* data, uint32_t num, uint32_t dim, const uint32_t* graph, uint32_t graph_degree,
                                       const float* centroids, uint32_t centroid_num, const uint32_t* start_points,
                                       const float* queries, uint32_t query_num, uint32_t top_k, uint32_t beam,
                                       uint32_t max_iterations, uint32_t min_iterations, uint32_t hash_bit,
                                       uint32_t hash_reset_interval, int metric, uint32_t* result_ids, float* result_dists,
                                       unsigned long long* counters, void* stream) {
    return launch_search(data, num, dim, graph, graph_degree, centroids, centroid_num, true, start_points, queries, query_num, top_k, beam,
                         max_iterations, min_iterations, hash_bit, hash_reset_interval, metric, result_ids, result_dists, counters, stream);
}

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
    if (graph_degree > 256 || beam > 512 || dim % 4 != 0 || dim > 4096 || top_k > beam || top_k > 128 || hash_bit < 1 || hash_bit > 13)
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
    const size_t lds_bytes = beam_lds_bytes(graph_degree) + 128 * 8 + (size_t{1} << hash_bit) * sizeof(uint32_t) + beam_stage_bytes(beam, beam == 512);
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
    if (graph_degree > 256 || beam > 512 || dim % 4 != 0 || dim > 4096 || top_k > beam || top_k > 128 || hash_bit < 1 || hash_bit > 13)
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
        const size_t lds_bytes = beam_lds_bytes(graph_degree) + 128 * 8 + (size_t{1} << hash_bit) * sizeof(uint32_t) + beam_stage_bytes(beam, beam == 512);
        GLIDE_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
        hipLaunchKernelGGL(fn, dim3(pairs), dim3(64), lds_bytes, s, a);
    }
    hipLaunchKernelGGL(merge_pairs_kernel, dim3(query_num), dim3(64), 0, s, segment_ids, pair_index, pair_dists, pair_ids, query_num, segment_num, top_k,
                       top_k <= 32 ? 32u : (top_k <= 64 ? 64u : 128u), final_dists, final_ids);
    return launch_status();
}
