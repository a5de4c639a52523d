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

template <int DIMV>
__device__ __forceinline__ uint32_t pick_centroid(uint32_t max_centroid, const RowRegs<DIMV>& q, const float* centroids,
                                                  uint32_t centroid_num, uint32_t dim, int metric, float* scratch, int lane) {
    switch (max_centroid) {  // bucket chosen like reference kernel_config.cuh:161-171
        case 32: return nearest_centroid<32, DIMV>(q, centroids, centroid_num, dim, metric, scratch, lane);
        case 64: return nearest_centroid<64, DIMV>(q, centroids, centroid_num, dim, metric, scratch, lane);
        case 128: return nearest_centroid<128, DIMV>(q, centroids, centroid_num, dim, metric, scratch, lane);
        default: return nearest_centroid<256, DIMV>(q, centroids, centroid_num, dim, metric, scratch, lane);
    }
}

template <int MAX_CAND, int MAX_BEAM, int DIMV>
__global__ __launch_bounds__(64) void search_kernel(SearchArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    auto* lds = reinterpret_cast<BeamLds<MAX_CAND>*>(smem);
    float* cent = reinterpret_cast<float*>(smem + sizeof(BeamLds<MAX_CAND>));
    uint32_t* hash = reinterpret_cast<uint32_t*>(cent + round_up32(a.centroid_num));
    const uint32_t qid = blockIdx.x;
    if (qid >= a.query_num) return;

    Beam<MAX_CAND, MAX_BEAM, DIMV> b;
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
}

using search_fn = void (*)(SearchArgs);

template <int MAX_CAND, int MAX_BEAM>
search_fn pick_dim(uint32_t dim) {
    if (dim <= 128) return search_kernel<MAX_CAND, MAX_BEAM, 1>;
    if (dim <= 256) return search_kernel<MAX_CAND, MAX_BEAM, 2>;
    if (dim <= 512) return search_kernel<MAX_CAND, MAX_BEAM, 4>;
    return search_kernel<MAX_CAND, MAX_BEAM, 8>;
}
template <int MAX_CAND>
search_fn pick_beam(uint32_t beam, uint32_t dim) {
    if (beam <= 64) return pick_dim<MAX_CAND, 64>(dim);
    if (beam <= 128) return pick_dim<MAX_CAND, 128>(dim);
    return pick_dim<MAX_CAND, 256>(dim);
}

}  // namespace glide

using namespace glide;

extern "C" int glide_hip_search(const float* data, uint32_t num, uint32_t dim, const uint32_t* graph, uint32_t graph_degree,
                                const float* centroids, uint32_t centroid_num, const uint32_t* start_points,
                                const float* queries, uint32_t query_num, uint32_t top_k, uint32_t beam,
                                uint32_t max_iterations, uint32_t min_iterations, uint32_t hash_bit,
                                uint32_t hash_reset_interval, int metric, uint32_t* result_ids, float* result_dists,
                                unsigned long long* counters, void* stream) {
    if (!data || !graph || !centroids || !start_points || !queries || !result_ids || !result_dists) return GLIDE_ERR_BAD_ARGUMENT;
    if (num == 0 || dim == 0 || graph_degree == 0 || centroid_num == 0 || beam == 0 || top_k == 0 || max_iterations == 0)
        return GLIDE_ERR_BAD_ARGUMENT;
    if (metric != GLIDE_METRIC_EUCLIDEAN && metric != GLIDE_METRIC_COSINE) return GLIDE_ERR_BAD_ARGUMENT;
    if (query_num == 0) return GLIDE_OK;
    if (graph_degree > 128 || beam > 256 || centroid_num > 256 || dim % 4 != 0 || dim > 1024 || top_k > beam ||
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

    const uint32_t max_cand = graph_degree <= 64 ? 64 : 128;
    search_fn fn = max_cand == 64 ? pick_beam<64>(beam, dim) : pick_beam<128>(beam, dim);
    const size_t lds_bytes = (max_cand == 64 ? sizeof(BeamLds<64>) : sizeof(BeamLds<128>)) +
                             round_up32(centroid_num) * sizeof(float) + (size_t{1} << hash_bit) * sizeof(uint32_t);
    hipLaunchKernelGGL(fn, dim3(query_num), dim3(64), lds_bytes, as_stream(stream), a);
    return launch_status();
}
