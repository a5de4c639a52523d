// Graph construction kernels: per-partition sub-graph build with pruning, cross-partition (boundary) merge,
// reverse-edge insertion and refinement.  One point per wavefront.
// Reference: graph_kernel.cuh (build_kernel :249-316, build_boundary_kernel :318-376, reverse_graph_kernel
// :378-414, insert_reverse_kernel :416-453, refine_kernel :580-673) as sequenced by glide_impl.cuh:77-316.
#include "prune.hpp"
#include "host_util.hpp"

namespace glide {

struct BuildArgs {
    const float* reorder_data;
    const uint32_t* knn_graph;
    const uint32_t* map;
    const uint32_t* segment_starts;
    const uint32_t* segment_lengths;
    const uint32_t* start_points;
    uint32_t* graph;
    unsigned long long* counters;
    uint32_t first_point, point_count;   // reorder ids [first_point, first_point + point_count)
    uint32_t segment_num, graph_degree;
    uint32_t boundary_start;             // boundary kernel: segment start (= num); 0xffffffff for the regular kernel
    uint32_t boundary_start_point;
    float relaxant;
    BeamParams p;                         // p.degree = knn_degree
};

template <int MAX_CAND, int MAX_BEAM, int DIMV>
__global__ __launch_bounds__(64) void build_kernel(BuildArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    auto* lds = reinterpret_cast<BeamLds<MAX_CAND>*>(smem);
    auto* pl = reinterpret_cast<PruneLds<MAX_BEAM>*>(smem + sizeof(BeamLds<MAX_CAND>));
    uint32_t* hash = reinterpret_cast<uint32_t*>(smem + sizeof(BeamLds<MAX_CAND>) + sizeof(PruneLds<MAX_BEAM>));
    if (blockIdx.x >= a.point_count) return;
    const uint32_t point = a.first_point + blockIdx.x;
    const bool boundary = a.boundary_start != kInvalid;

    const bool segment_mode = a.map == nullptr;   // one staged partition: local ids in and out (build_for_large_kernel)
    uint32_t seg_start, entry;
    if (segment_mode) {
        seg_start = 0;
        entry = a.boundary_start_point;
    } else if (boundary) {
        seg_start = a.boundary_start;
        entry = a.boundary_start_point;
    } else {
        uint32_t seg = 0;
        for (; seg < a.segment_num; seg++)
            if (point < a.segment_starts[seg] + a.segment_lengths[seg]) break;
        seg_start = a.segment_starts[seg];
        entry = a.start_points[seg];
    }
    const float* sdata = a.reorder_data + static_cast<size_t>(seg_start) * a.p.dim;
    const uint32_t* sgraph = a.knn_graph + static_cast<size_t>(seg_start) * a.p.degree;

    Beam<MAX_CAND, MAX_BEAM, DIMV> b;
    b.init(lds, hash, a.p, a.reorder_data + static_cast<size_t>(point) * a.p.dim);
    // get_init (search_kernel.cuh:336-360): all neighbours of the entry are hashed; the one whose *local* id equals
    // this point's *reorder* id is left unscored (the reference compares across id spaces, graph_kernel.cuh:295-298)
    b.expand(entry, sgraph, sdata, kInvalid, point);
    b.run(sgraph, sdata, point - seg_start);

    uint32_t pool = beam_to_pool(b, pl);
    prune_pool<MAX_BEAM, DIMV>(pl, pool, a.reorder_data, a.p.dim, seg_start, a.graph_degree, a.relaxant, a.p.metric, b.lane,
                               b.cnt.rows_scored);
    wave_sync();
    if (segment_mode) {   // map_to_graph (graph_kernel.cuh:145-150)
        uint32_t* row = a.graph + static_cast<size_t>(point) * a.graph_degree;
        for (uint32_t i = b.lane; i < a.graph_degree; i += 64) row[i] = pl->neighbor[i];
        b.flush_counters(a.counters);
        return;
    }
    uint32_t* row = a.graph + static_cast<size_t>(a.map[point]) * a.graph_degree;
    if (boundary) {
        merge_boundary_row<MAX_BEAM>(pl, row, a.map, a.graph_degree, b.lane);
    } else {  // map_to_graph_sub (graph_kernel.cuh:152-158)
        for (uint32_t i = b.lane; i < a.graph_degree; i += 64) {
            const uint32_t nb = pl->neighbor[i];
            row[i] = nb == kInvalid ? kInvalid : a.map[nb];
        }
    }
    b.flush_counters(a.counters);
}

struct RefineArgs {
    const float* data;
    const uint32_t* graph_in;
    uint32_t* graph_out;
    const float* centroids;
    const uint32_t* start_points;
    unsigned long long* counters;
    const uint32_t* order;   // nullable: workgroup i refines point order[i] (a permutation of the points)
    uint32_t num, centroid_num, max_centroid, segment_start_point;
    float relaxant;
    BeamParams p;   // p.degree = graph_degree
};

template <int DIMV>
__device__ __forceinline__ uint32_t pick_centroid_refine(uint32_t max_centroid, const RowRegs<DIMV>& q, const float* centroids,
                                                         uint32_t centroid_num, uint32_t dim, int metric, float* scratch, int lane) {
    switch (max_centroid) {
        case 32: return nearest_centroid<32, DIMV>(q, centroids, centroid_num, dim, metric, scratch, lane);
        case 64: return nearest_centroid<64, DIMV>(q, centroids, centroid_num, dim, metric, scratch, lane);
        case 128: return nearest_centroid<128, DIMV>(q, centroids, centroid_num, dim, metric, scratch, lane);
        default: return nearest_centroid<256, DIMV>(q, centroids, centroid_num, dim, metric, scratch, lane);
    }
}

// Rows are read from graph_in and written to graph_out (every row is written: copied, with its empty slots
// filled).  The reference refines in place while other blocks still traverse the rows.
template <int MAX_CAND, int MAX_BEAM, int DIMV>
__global__ __launch_bounds__(64) void refine_kernel(RefineArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    auto* lds = reinterpret_cast<BeamLds<MAX_CAND>*>(smem);
    using Prune = PruneLds<MAX_BEAM, (MAX_CAND < 64 ? 64 : MAX_CAND)>;   // the row has at most MAX_CAND slots here
    auto* pl = reinterpret_cast<Prune*>(smem + sizeof(BeamLds<MAX_CAND>));
    float* cent = reinterpret_cast<float*>(smem + sizeof(BeamLds<MAX_CAND>) + sizeof(Prune));
    uint32_t* hash = reinterpret_cast<uint32_t*>(cent + round_up32(a.centroid_num));
    if (blockIdx.x >= a.num) return;
    const uint32_t point = a.order ? a.order[blockIdx.x] : blockIdx.x;
    if (point >= a.num) return;
    const int lane = lane_id();
    const uint32_t D = a.p.degree;
    const uint32_t* in_row = a.graph_in + static_cast<size_t>(point) * D;
    uint32_t* out_row = a.graph_out + static_cast<size_t>(point) * D;

    uint32_t need = 0;
    for (uint32_t base = 0; base < Prune::kCap; base += 64) {
        const uint32_t i = base + lane;
        const uint32_t g = i < D ? in_row[i] : kInvalid;
        pl->s_graph[i] = g;
        if (i < D) out_row[i] = g;
        need += __popcll(ballot(i < D && g == kInvalid));
    }
    wave_sync();
    if (need == 0) return;

    Beam<MAX_CAND, MAX_BEAM, DIMV> b;
    b.init(lds, hash, a.p, a.data + static_cast<size_t>(point) * a.p.dim);
    if (a.centroids != nullptr) {
        const uint32_t c0 = pick_centroid_refine<DIMV>(a.max_centroid, b.q, a.centroids, a.centroid_num, a.p.dim, a.p.metric, cent, lane);
        b.expand(a.start_points[c0], a.graph_in, a.data, kInvalid, kInvalid);
    } else {   // refine_for_large_kernel (graph_kernel.cuh:796-798): get_init from the segment's start point
        b.expand(a.segment_start_point, a.graph_in, a.data, kInvalid, point);
    }
    b.run(a.graph_in, a.data, point);

    uint32_t pool = beam_to_pool(b, pl);
    prune_pool_refine<MAX_BEAM, DIMV>(pl, pool, a.data, a.p.dim, point, D, need, a.relaxant, a.p.metric, lane, b.cnt.rows_scored);
    wave_sync();
    uint32_t used = 0;
    for (uint32_t base = 0; base < round_up32(D); base += 64) {  // holes in slot order (graph_kernel.cuh:659-671)
        const uint32_t i = base + lane;
        const bool hole = i < D && pl->s_graph[i] == kInvalid;
        const uint64_t m = ballot(hole);
        if (hole) out_row[i] = pl->neighbor[used + prefix_count(m)];
        used += __popcll(m);
    }
    b.flush_counters(a.counters);
}

// ------------------------------------------------------------------------------------------ reverse edges
// Reference order of arrival in a row's reverse list is whatever the atomics give; here the list is the D
// smallest (column, source) pairs, i.e. the order of a sequential sweep over columns then sources.
//
// pass 1: one wavefront per source s.  For each column c with target t = graph[s][c] < num, the row of t is read
// coalesced and searched for s.  Missing pairs are counted per target and remembered in a bit per (s, c).
__global__ __launch_bounds__(256) void reverse_count_kernel(const uint32_t* graph, uint32_t num, uint32_t D, uint32_t* miss_bits,
                                                            uint32_t* counts) {
    const int lane = lane_id();
    const uint32_t s = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (s >= num) return;
    const uint32_t words = ceil_div(D, 32);
    for (uint32_t cb = 0; cb < D; cb += 32) {
        uint32_t bits = 0;
        const uint32_t cend = cb + 32 < D ? cb + 32 : D;
        for (uint32_t c = cb; c < cend; c++) {
            const uint32_t t = graph[static_cast<size_t>(s) * D + c];   // wave-uniform
            if (t >= num) continue;
            bool have = false;
            for (uint32_t i = lane; i < D; i += 64) have |= graph[static_cast<size_t>(t) * D + i] == s;
            if (ballot(have) == 0) {
                bits |= 1u << (c - cb);
                if (lane == 0) atomicAdd(&counts[t], 1u);
            }
        }
        if (lane == 0) miss_bits[static_cast<size_t>(s) * words + cb / 32] = bits;
    }
}

// pass 2: bucket offsets (any order; only the bucket contents matter)
__global__ void reverse_offsets_kernel(const uint32_t* counts, uint32_t num, uint32_t* offsets, unsigned long long* cursor) {
    const uint32_t t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= num) return;
    const uint32_t c = counts[t];
    offsets[t] = c ? static_cast<uint32_t>(atomicAdd(cursor, static_cast<unsigned long long>(c))) : 0u;
}

// pass 3: scatter (column, source) keys into the target's bucket
__global__ void reverse_scatter_kernel(const uint32_t* graph, uint32_t num, uint32_t D, const uint32_t* miss_bits,
                                       const uint32_t* offsets, uint32_t* fill, unsigned long long* pool) {
    const uint32_t s = blockIdx.x * blockDim.x + threadIdx.x;
    if (s >= num) return;
    const uint32_t words = ceil_div(D, 32);
    for (uint32_t w = 0; w < words; w++) {
        uint32_t bits = miss_bits[static_cast<size_t>(s) * words + w];
        while (bits) {
            const uint32_t c = w * 32 + __builtin_ctz(bits);
            bits &= bits - 1;
            const uint32_t t = graph[static_cast<size_t>(s) * D + c];
            const uint32_t pos = atomicAdd(&fill[t], 1u);
            pool[static_cast<size_t>(offsets[t]) + pos] = (static_cast<unsigned long long>(c) << 32) | s;
        }
    }
}

// pass 4: one wavefront per target: the min(count, D) smallest keys of its bucket, ascending -> reverse list
__global__ __launch_bounds__(256) void reverse_select_kernel(uint32_t num, uint32_t D, const uint32_t* counts, const uint32_t* offsets,
                                                             const unsigned long long* pool, uint32_t* reverse_graph) {
    const int lane = lane_id();
    const uint32_t t = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= num) return;
    const uint32_t cnt = counts[t];
    const uint32_t take = cnt < D ? cnt : D;
    const unsigned long long* bucket = pool + offsets[t];
    unsigned long long last = 0;
    bool have_last = false;
    for (uint32_t k = 0; k < take; k++) {
        unsigned long long best = ~0ull;
        for (uint32_t i = lane; i < cnt; i += 64) {
            const unsigned long long key = bucket[i];
            if ((!have_last || key > last) && key < best) best = key;
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            const unsigned long long o = __shfl_xor(best, off);
            best = o < best ? o : best;
        }
        last = best;
        have_last = true;
        if (lane == 0) reverse_graph[static_cast<size_t>(t) * D + k] = static_cast<uint32_t>(best & 0xffffffffull);
    }
    for (uint32_t k = take + lane; k < D; k += 64) reverse_graph[static_cast<size_t>(t) * D + k] = kInvalid;
}

// insert_reverse_kernel (graph_kernel.cuh:416-453): empty slots, in order, take the first reverse edges
__global__ __launch_bounds__(256) void insert_reverse_kernel(uint32_t* graph, const uint32_t* reverse_graph, const uint32_t* counts,
                                                             uint32_t num, uint32_t D) {
    const int lane = lane_id();
    const uint32_t p = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (p >= num) return;
    const uint32_t nrev = counts[p] > D ? D : counts[p];
    uint32_t used = 0;
    for (uint32_t base = 0; base < D && used < nrev; base += 64) {
        const uint32_t i = base + lane;
        const bool hole = i < D && graph[static_cast<size_t>(p) * D + i] == kInvalid;
        const uint64_t m = ballot(hole);
        const uint32_t pos = used + prefix_count(m);
        if (hole && pos < nrev) graph[static_cast<size_t>(p) * D + i] = reverse_graph[static_cast<size_t>(p) * D + pos];
        used += __popcll(m);
    }
}

// ------------------------------------------------------------------------------------------ merged large build
// A staged partition's sub-graph holds partition-local ids.  Its rows go to rows segment_start .. of the merged graph
// with segment_start added to every id (what map_to_graph does through `map` on the small path,
// graph_kernel.cuh:145-150; here the merged graph stays in reorder-id space, so the map is an offset).
__global__ __launch_bounds__(256) void place_segment_kernel(const uint32_t* segment_graph, size_t words, uint32_t segment_start, uint32_t* merged) {
    const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= words) return;
    const uint32_t v = segment_graph[i];
    merged[i] = v == kInvalid ? kInvalid : v + segment_start;
}

// map_to_graph_boundary (graph_kernel.cuh:160-247) as a pass of its own: boundary copy i found the neighbours
// boundary_graph[i] (ids local to the boundary segment); they are merged into the row of the point it is a copy of,
// home_rows[i], every neighbour l being named by its own home row home_rows[l].  One wavefront per boundary copy.
__global__ __launch_bounds__(64) void merge_boundary_kernel(const uint32_t* boundary_graph, uint32_t boundary_num, uint32_t D,
                                                            const uint32_t* home_rows, uint32_t* merged) {
    __shared__ PruneLds<64> pl;
    const uint32_t i = blockIdx.x;
    if (i >= boundary_num) return;
    const int lane = lane_id();
    for (uint32_t j = lane; j < kMaxDegree; j += 64) pl.neighbor[j] = j < D ? boundary_graph[static_cast<size_t>(i) * D + j] : kInvalid;
    wave_sync();
    merge_boundary_row<64>(&pl, merged + static_cast<size_t>(home_rows[i]) * D, home_rows, D, lane);
}

// ------------------------------------------------------------------------------------------ dispatch
using build_fn = void (*)(BuildArgs);
using refine_fn = void (*)(RefineArgs);

template <int MAX_CAND, int MAX_BEAM>
build_fn pick_build_dim(uint32_t dim) {
    if (dim <= 128) return build_kernel<MAX_CAND, MAX_BEAM, 1>;
    if (dim <= 256) return build_kernel<MAX_CAND, MAX_BEAM, 2>;
    if (dim <= 512) return build_kernel<MAX_CAND, MAX_BEAM, 4>;
    if (dim <= 1024) return build_kernel<MAX_CAND, MAX_BEAM, 8>;
    if (dim <= 2048) return build_kernel<MAX_CAND, MAX_BEAM, 16>;
    return build_kernel<MAX_CAND, MAX_BEAM, 32>;
}
template <int MAX_CAND>
build_fn pick_build_beam(uint32_t beam, uint32_t dim) {
    if (beam <= 64) return pick_build_dim<MAX_CAND, 64>(dim);
    if (beam <= 128) return pick_build_dim<MAX_CAND, 128>(dim);
    if (beam <= 256) return pick_build_dim<MAX_CAND, 256>(dim);
    return pick_build_dim<MAX_CAND, 512>(dim);
}
template <int MAX_CAND, int MAX_BEAM>
refine_fn pick_refine_dim(uint32_t dim) {
    if (dim <= 128) return refine_kernel<MAX_CAND, MAX_BEAM, 1>;
    if (dim <= 256) return refine_kernel<MAX_CAND, MAX_BEAM, 2>;
    if (dim <= 512) return refine_kernel<MAX_CAND, MAX_BEAM, 4>;
    if (dim <= 1024) return refine_kernel<MAX_CAND, MAX_BEAM, 8>;
    if (dim <= 2048) return refine_kernel<MAX_CAND, MAX_BEAM, 16>;
    return refine_kernel<MAX_CAND, MAX_BEAM, 32>;
}
template <int MAX_CAND>
refine_fn pick_refine_beam(uint32_t beam, uint32_t dim) {
    if (beam <= 64) return pick_refine_dim<MAX_CAND, 64>(dim);
    if (beam <= 128) return pick_refine_dim<MAX_CAND, 128>(dim);
    if (beam <= 256) return pick_refine_dim<MAX_CAND, 256>(dim);
    return pick_refine_dim<MAX_CAND, 512>(dim);
}

size_t prune_lds_bytes(uint32_t beam) {
    return beam <= 64 ? sizeof(PruneLds<64>) : beam <= 128 ? sizeof(PruneLds<128>) : beam <= 256 ? sizeof(PruneLds<256>) : sizeof(PruneLds<512>);
}
// the refine kernel's layout: row arrays sized by the degree bucket instead of the maximum degree
template <int CAP>
size_t prune_lds_bytes_cap(uint32_t beam) {
    return beam <= 64 ? sizeof(PruneLds<64, CAP>) : beam <= 128 ? sizeof(PruneLds<128, CAP>) : beam <= 256 ? sizeof(PruneLds<256, CAP>)
                                                                                                          : sizeof(PruneLds<512, CAP>);
}
size_t prune_lds_bytes_refine(uint32_t beam, uint32_t degree) {
    return degree <= 64 ? prune_lds_bytes_cap<64>(beam) : degree <= 128 ? prune_lds_bytes_cap<128>(beam) : prune_lds_bytes_cap<256>(beam);
}

int check_beam_sizes(uint32_t degree, uint32_t graph_degree, uint32_t beam, uint32_t dim, uint32_t hash_bit, int metric) {
    if (degree == 0 || graph_degree == 0 || beam == 0 || dim == 0) return GLIDE_ERR_BAD_ARGUMENT;
    if (metric != GLIDE_METRIC_EUCLIDEAN && metric != GLIDE_METRIC_COSINE) return GLIDE_ERR_BAD_ARGUMENT;
    if (degree > kMaxDegree || graph_degree > kMaxDegree || !beam_supported(beam) || dim % 4 != 0 || dim > 4096 || hash_bit < 1 || hash_bit > 13)
        return GLIDE_ERR_UNSUPPORTED;
    return GLIDE_OK;
}

int launch_build(BuildArgs& a, hipStream_t stream) {
    build_fn fn = a.p.degree <= 64 ? pick_build_beam<64>(a.p.beam, a.p.dim)
                : a.p.degree <= 128 ? pick_build_beam<128>(a.p.beam, a.p.dim) : pick_build_beam<256>(a.p.beam, a.p.dim);
    const size_t lds_bytes = beam_lds_bytes(a.p.degree) + prune_lds_bytes(a.p.beam) + (size_t{1} << a.p.hash_bit) * sizeof(uint32_t);
    GLIDE_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
    hipLaunchKernelGGL(fn, dim3(a.point_count), dim3(64), lds_bytes, stream, a);
    return launch_status();
}

}  // namespace glide

using namespace glide;

extern "C" {

int glide_hip_build_subgraph(const float* reorder_data, uint32_t num, uint32_t dim, const uint32_t* knn_graph, uint32_t knn_degree,
                             const uint32_t* map, const uint32_t* segment_starts, const uint32_t* segment_lengths,
                             uint32_t segment_num, const uint32_t* start_points, uint32_t graph_degree, uint32_t beam,
                             uint32_t max_iterations, uint32_t min_iterations, uint32_t hash_bit, uint32_t hash_reset_interval,
                             float relaxant, int metric, uint32_t* graph, unsigned long long* counters, void* stream) {
    if (!reorder_data || !knn_graph || !map || !segment_starts || !segment_lengths || !start_points || !graph)
        return GLIDE_ERR_BAD_ARGUMENT;
    if (max_iterations == 0 || segment_num == 0) return GLIDE_ERR_BAD_ARGUMENT;
    int rc = check_beam_sizes(knn_degree, graph_degree, beam, dim, hash_bit, metric);
    if (rc != GLIDE_OK) return rc;
    if (num == 0) return GLIDE_OK;
    BuildArgs a;
    a.reorder_data = reorder_data;
    a.knn_graph = knn_graph;
    a.map = map;
    a.segment_starts = segment_starts;
    a.segment_lengths = segment_lengths;
    a.start_points = start_points;
    a.graph = graph;
    a.counters = counters;
    a.first_point = 0;
    a.point_count = num;
    a.segment_num = segment_num;
    a.graph_degree = graph_degree;
    a.boundary_start = kInvalid;
    a.boundary_start_point = 0;
    a.relaxant = relaxant;
    a.p = BeamParams{beam, knn_degree, dim, hash_bit, hash_reset_interval ? hash_reset_interval : 1, max_iterations, min_iterations, metric};
    return launch_build(a, as_stream(stream));
}

int glide_hip_build_boundary(const float* reorder_data, uint32_t num, uint32_t reorder_num, uint32_t dim, const uint32_t* knn_graph,
                             uint32_t knn_degree, const uint32_t* map, uint32_t start_point, uint32_t graph_degree, uint32_t beam,
                             uint32_t max_iterations, uint32_t min_iterations, uint32_t hash_bit, uint32_t hash_reset_interval,
                             float relaxant, int metric, uint32_t* graph, unsigned long long* counters, void* stream) {
    if (!reorder_data || !knn_graph || !map || !graph) return GLIDE_ERR_BAD_ARGUMENT;
    if (max_iterations == 0 || reorder_num < num) return GLIDE_ERR_BAD_ARGUMENT;
    int rc = check_beam_sizes(knn_degree, graph_degree, beam, dim, hash_bit, metric);
    if (rc != GLIDE_OK) return rc;
    if (reorder_num == num) return GLIDE_OK;
    if (start_point >= reorder_num - num) return GLIDE_ERR_BAD_ARGUMENT;
    BuildArgs a;
    a.reorder_data = reorder_data;
    a.knn_graph = knn_graph;
    a.map = map;
    a.segment_starts = nullptr;
    a.segment_lengths = nullptr;
    a.start_points = nullptr;
    a.graph = graph;
    a.counters = counters;
    a.first_point = num;
    a.point_count = reorder_num - num;
    a.segment_num = 0;
    a.graph_degree = graph_degree;
    a.boundary_start = num;
    a.boundary_start_point = start_point;
    a.relaxant = relaxant;
    a.p = BeamParams{beam, knn_degree, dim, hash_bit, hash_reset_interval ? hash_reset_interval : 1, max_iterations, min_iterations, metric};
    return launch_build(a, as_stream(stream));
}

int glide_hip_build_segment(const float* segment_data, uint32_t num, uint32_t dim, const uint32_t* knn_graph, uint32_t knn_degree,
                            uint32_t start_point, uint32_t graph_degree, uint32_t beam, uint32_t max_iterations, uint32_t min_iterations,
                            uint32_t hash_bit, uint32_t hash_reset_interval, float relaxant, int metric, uint32_t* graph,
                            unsigned long long* counters, void* stream) {
    if (!segment_data || !knn_graph || !graph) return GLIDE_ERR_BAD_ARGUMENT;
    if (max_iterations == 0) return GLIDE_ERR_BAD_ARGUMENT;
    int rc = check_beam_sizes(knn_degree, graph_degree, beam, dim, hash_bit, metric);
    if (rc != GLIDE_OK) return rc;
    if (num == 0) return GLIDE_OK;
    if (start_point >= num) return GLIDE_ERR_BAD_ARGUMENT;
    BuildArgs a;
    a.reorder_data = segment_data;
    a.knn_graph = knn_graph;
    a.map = nullptr;
    a.segment_starts = nullptr;
    a.segment_lengths = nullptr;
    a.start_points = nullptr;
    a.graph = graph;
    a.counters = counters;
    a.first_point = 0;
    a.point_count = num;
    a.segment_num = 0;
    a.graph_degree = graph_degree;
    a.boundary_start = kInvalid;
    a.boundary_start_point = start_point;
    a.relaxant = relaxant;
    a.p = BeamParams{beam, knn_degree, dim, hash_bit, hash_reset_interval ? hash_reset_interval : 1, max_iterations, min_iterations, metric};
    return launch_build(a, as_stream(stream));
}

int glide_hip_refine_segment(const float* segment_data, uint32_t num, uint32_t dim, const uint32_t* graph_in, uint32_t* graph_out,
                             uint32_t graph_degree, uint32_t start_point, uint32_t beam, uint32_t max_iterations, uint32_t min_iterations,
                             uint32_t hash_bit, uint32_t hash_reset_interval, float relaxant, int metric, unsigned long long* counters,
                             void* stream) {
    if (!segment_data || !graph_in || !graph_out || graph_in == graph_out) return GLIDE_ERR_BAD_ARGUMENT;
    if (max_iterations == 0) return GLIDE_ERR_BAD_ARGUMENT;
    int rc = check_beam_sizes(graph_degree, graph_degree, beam, dim, hash_bit, metric);
    if (rc != GLIDE_OK) return rc;
    if (num == 0) return GLIDE_OK;
    if (start_point >= num) return GLIDE_ERR_BAD_ARGUMENT;
    RefineArgs a;
    a.order = nullptr;
    a.data = segment_data;
    a.graph_in = graph_in;
    a.graph_out = graph_out;
    a.centroids = nullptr;
    a.start_points = nullptr;
    a.counters = counters;
    a.num = num;
    a.centroid_num = 0;
    a.max_centroid = 32;
    a.segment_start_point = start_point;
    a.relaxant = relaxant;
    a.p = BeamParams{beam, graph_degree, dim, hash_bit, hash_reset_interval ? hash_reset_interval : 1, max_iterations, min_iterations, metric};
    refine_fn fn = graph_degree <= 64 ? pick_refine_beam<64>(beam, dim)
                 : graph_degree <= 128 ? pick_refine_beam<128>(beam, dim) : pick_refine_beam<256>(beam, dim);
    const size_t lds_bytes = beam_lds_bytes(graph_degree) + prune_lds_bytes(beam) + (size_t{1} << hash_bit) * sizeof(uint32_t);
    GLIDE_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
    hipLaunchKernelGGL(fn, dim3(num), dim3(64), lds_bytes, as_stream(stream), a);
    return launch_status();
}

size_t glide_hip_reverse_edges_workspace_bytes(uint32_t num, uint32_t graph_degree) {
    const size_t n = num, words = ceil_div(graph_degree, 32);
    // miss bits + offsets + fill (u32 each), cursor (u64, 256-byte slot), pool of (column, source) keys
    return n * words * 4 + n * 4 + n * 4 + 256 + n * graph_degree * 8;
}

int glide_hip_reverse_edges(const uint32_t* graph, uint32_t num, uint32_t graph_degree, uint32_t* reverse_graph,
                            uint32_t* reverse_counts, void* workspace, size_t workspace_bytes, void* stream) {
    if (!graph || !reverse_graph || !reverse_counts || !workspace) return GLIDE_ERR_BAD_ARGUMENT;
    if (graph_degree == 0) return GLIDE_ERR_BAD_ARGUMENT;
    if (graph_degree > 256) return GLIDE_ERR_UNSUPPORTED;
    if (num == 0) return GLIDE_OK;
    if (workspace_bytes < glide_hip_reverse_edges_workspace_bytes(num, graph_degree) || reinterpret_cast<uintptr_t>(workspace) % 8)
        return GLIDE_ERR_BAD_ARGUMENT;
    hipStream_t s = as_stream(stream);
    const size_t n = num, words = ceil_div(graph_degree, 32);
    unsigned char* w = static_cast<unsigned char*>(workspace);
    unsigned long long* cursor = reinterpret_cast<unsigned long long*>(w);
    unsigned long long* pool = reinterpret_cast<unsigned long long*>(w + 256);
    uint32_t* offsets = reinterpret_cast<uint32_t*>(w + 256 + n * graph_degree * 8);
    uint32_t* fill = offsets + n;
    uint32_t* miss = fill + n;
    int rc = glide_hip_fill_u32(reverse_counts, 0u, n, stream);
    if (rc == GLIDE_OK) rc = glide_hip_fill_u32(fill, 0u, n, stream);
    if (rc == GLIDE_OK) rc = glide_hip_fill_u32(reinterpret_cast<uint32_t*>(cursor), 0u, 2, stream);
    if (rc != GLIDE_OK) return rc;
    hipLaunchKernelGGL(reverse_count_kernel, dim3(ceil_div(num, 4)), dim3(256), 0, s, graph, num, graph_degree, miss, reverse_counts);
    hipLaunchKernelGGL(reverse_offsets_kernel, dim3(ceil_div(num, 256)), dim3(256), 0, s, reverse_counts, num, offsets, cursor);
    hipLaunchKernelGGL(reverse_scatter_kernel, dim3(ceil_div(num, 256)), dim3(256), 0, s, graph, num, graph_degree, miss, offsets, fill, pool);
    hipLaunchKernelGGL(reverse_select_kernel, dim3(ceil_div(num, 4)), dim3(256), 0, s, num, graph_degree, reverse_counts, offsets, pool,
                       reverse_graph);
    (void) words;
    return launch_status();
}

int glide_hip_insert_reverse(uint32_t* graph, const uint32_t* reverse_graph, const uint32_t* reverse_counts, uint32_t num,
                             uint32_t graph_degree, void* stream) {
    if (!graph || !reverse_graph || !reverse_counts || graph_degree == 0) return GLIDE_ERR_BAD_ARGUMENT;
    if (num == 0) return GLIDE_OK;
    hipLaunchKernelGGL(insert_reverse_kernel, dim3(ceil_div(num, 4)), dim3(256), 0, as_stream(stream), graph, reverse_graph,
                       reverse_counts, num, graph_degree);
    return launch_status();
}

int glide_hip_place_segment_graph(const uint32_t* segment_graph, uint32_t segment_length, uint32_t graph_degree, uint32_t segment_start,
                                  uint32_t* merged_graph, void* stream) {
    if (!segment_graph || !merged_graph || graph_degree == 0) return GLIDE_ERR_BAD_ARGUMENT;
    if (segment_length == 0) return GLIDE_OK;
    const size_t words = static_cast<size_t>(segment_length) * graph_degree;
    uint32_t* dst = merged_graph + static_cast<size_t>(segment_start) * graph_degree;
    hipLaunchKernelGGL(place_segment_kernel, dim3(static_cast<uint32_t>((words + 255) / 256)), dim3(256), 0, as_stream(stream), segment_graph, words,
                       segment_start, dst);
    return launch_status();
}

int glide_hip_merge_boundary_graph(const uint32_t* boundary_graph, uint32_t boundary_num, uint32_t graph_degree, const uint32_t* home_rows,
                                   uint32_t* merged_graph, void* stream) {
    if (!boundary_graph || !home_rows || !merged_graph || graph_degree == 0) return GLIDE_ERR_BAD_ARGUMENT;
    if (graph_degree > kMaxDegree) return GLIDE_ERR_UNSUPPORTED;
    if (boundary_num == 0) return GLIDE_OK;
    hipLaunchKernelGGL(merge_boundary_kernel, dim3(boundary_num), dim3(64), 0, as_stream(stream), boundary_graph, boundary_num, graph_degree,
                       home_rows, merged_graph);
    return launch_status();
}

}  // extern "C"

namespace {
int launch_refine(const float* data, uint32_t num, uint32_t dim, const uint32_t* graph_in, uint32_t* graph_out, uint32_t graph_degree,
                  const float* centroids, uint32_t centroid_num, bool rank_all_centroids, const uint32_t* start_points, uint32_t beam,
                  uint32_t max_iterations, uint32_t min_iterations, uint32_t hash_bit, uint32_t hash_reset_interval, float relaxant, int metric,
                  const uint32_t* order, unsigned long long* counters, void* stream) {
    if (!data || !graph_in || !graph_out || !centroids || !start_points || graph_in == graph_out) return GLIDE_ERR_BAD_ARGUMENT;
    if (max_iterations == 0 || centroid_num == 0) return GLIDE_ERR_BAD_ARGUMENT;
    int rc = check_beam_sizes(graph_degree, graph_degree, beam, dim, hash_bit, metric);
    if (rc != GLIDE_OK) return rc;
    if (centroid_num > 256) return GLIDE_ERR_UNSUPPORTED;
    if (num == 0) return GLIDE_OK;
    RefineArgs a;
    a.data = data;
    a.graph_in = graph_in;
    a.graph_out = graph_out;
    a.centroids = centroids;
    a.start_points = start_points;
    a.counters = counters;
    a.order = order;
    a.num = num;
    a.centroid_num = centroid_num;
    a.max_centroid = centroid_num <= 32 ? 32 : (graph_degree <= 64 ? 64 : (graph_degree <= 128 ? 128 : 256));
    if (rank_all_centroids) a.max_centroid = centroid_num <= 32 ? 32 : (centroid_num <= 64 ? 64 : (centroid_num <= 128 ? 128 : 256));
    a.segment_start_point = 0;
    a.relaxant = relaxant;
    a.p = BeamParams{beam, graph_degree, dim, hash_bit, hash_reset_interval ? hash_reset_interval : 1, max_iterations, min_iterations, metric};
    refine_fn fn = graph_degree <= 64 ? pick_refine_beam<64>(beam, dim)
                 : graph_degree <= 128 ? pick_refine_beam<128>(beam, dim) : pick_refine_beam<256>(beam, dim);
    const size_t lds_bytes = beam_lds_bytes(graph_degree) + prune_lds_bytes_refine(beam, graph_degree) + round_up32(centroid_num) * sizeof(float) +
                             (size_t{1} << hash_bit) * sizeof(uint32_t);
    GLIDE_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
    hipLaunchKernelGGL(fn, dim3(num), dim3(64), lds_bytes, as_stream(stream), a);
    return launch_status();
}
}  // namespace

extern "C" int glide_hip_refine(const float* data, uint32_t num, uint32_t dim, const uint32_t* graph_in, uint32_t* graph_out,
                                uint32_t graph_degree, const float* centroids, uint32_t centroid_num, const uint32_t* start_points,
                                uint32_t beam, uint32_t max_iterations, uint32_t min_iterations, uint32_t hash_bit,
                                uint32_t hash_reset_interval, float relaxant, int metric, const uint32_t* order,
                                unsigned long long* counters, void* stream) {
    return launch_refine(data, num, dim, graph_in, graph_out, graph_degree, centroids, centroid_num, false, start_points, beam, max_iterations,
                         min_iterations, hash_bit, hash_reset_interval, relaxant, metric, order, counters, stream);
}

extern "C" int glide_hip_refine_merged(const float* data, uint32_t num, uint32_t dim, const uint32_t* graph_in, uint32_t* graph_out,
                                       uint32_t graph_degree, const float* centroids, uint32_t centroid_num, const uint32_t* start_points,
                                       uint32_t beam, uint32_t max_iterations, uint32_t min_iterations, uint32_t hash_bit,
                                       uint32_t hash_reset_interval, float relaxant, int metric, const uint32_t* order,
                                       unsigned long long* counters, void* stream) {
    return launch_refine(data, num, dim, graph_in, graph_out, graph_degree, centroids, centroid_num, true, start_points, beam, max_iterations,
                         min_iterations, hash_bit, hash_reset_interval, relaxant, metric, order, counters, stream);
}
