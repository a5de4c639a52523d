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

// Beams above 256 on rows of up to 512 dims: held to the registers of four wavefronts per SIMD (the kernel asks for a
// dozen more, which costs it the fourth wavefront and buys nothing: the vector ALU is the limit).
template <int MAX_CAND, int MAX_BEAM, int DIMV, bool WHOLE = false>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(MAX_BEAM > 256 && DIMV <= 4 ? 4 : 1)))
void search_kernel(SearchArgs a) {
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

using search_fn = void (*)(SearchArgs);

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
    if (graph_degree > 256 || !beam_supported(beam) || centroid_num > 256 || dim % 4 != 0 || dim > 4096 || top_k > beam ||
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
                             (size_t{1} << hash_bit) * sizeof(uint32_t) +
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
