// Relaxed-RNG pruning of a finished beam, boundary merge and hole filling for one wavefront.
// Reference: sync_prune (graph_kernel.cuh:70-143), select_point + sync_prune_refine (:455-578),
// map_to_graph_boundary (:160-247).
#pragma once
#include "beam.hpp"

namespace glide {

constexpr uint32_t kMaxDegree = 256;   // largest graph / kNN degree (reference kernel_config.cuh:53-60)

// DCAP = capacity of the per-row arrays: a multiple of 64 that is at least round_up32(graph_degree).  The refine kernel
// sizes it by its degree bucket (less LDS per wavefront, more wavefronts per CU); the build kernels, whose output
// degree is independent of the degree bucket of the kNN graph they search, keep the maximum.
template <int MAX_BEAM, int DCAP = static_cast<int>(kMaxDegree)>
struct PruneLds {
    static_assert(DCAP % 64 == 0 && DCAP <= static_cast<int>(kMaxDegree), "row capacity");
    static constexpr uint32_t kCap = DCAP;
    uint32_t pool_id[MAX_BEAM];
    float pool_dist[MAX_BEAM];
    uint32_t keep[MAX_BEAM];
    uint32_t neighbor[DCAP];
    uint32_t s_graph[DCAP];
    uint32_t fresh[DCAP];
    uint32_t dup_mask[DCAP / 32];
};

// Beam registers -> LDS pool in rank order with the explored bit stripped (graph_kernel.cuh:65-67), dropping
// slots that never held a node (their id would be dereferenced by the reference).  Returns the pool size.
template <int MAX_CAND, int MAX_BEAM, int DIMV, class PL>
__device__ __forceinline__ uint32_t beam_to_pool(Beam<MAX_CAND, MAX_BEAM, DIMV>& b, PL* pl) {
    constexpr int NB = MAX_BEAM / 64;
    // rank order is e = NB*lane + r; compact register by register would break the order, so stage then compact
#pragma unroll
    for (int r = 0; r < NB; r++) {
        const uint32_t e = NB * b.lane + r;
        pl->keep[e] = b.bv[r] & kClean;                       // reuse `keep` as staging for ids
        pl->pool_dist[e] = b.bk[r];
    }
    wave_sync();
    uint32_t n = 0;
    for (uint32_t base = 0; base < b.p.beam; base += 64) {
        const uint32_t i = base + b.lane;
        const uint32_t id = i < b.p.beam ? pl->keep[i] : kClean;
        const float d = i < b.p.beam ? pl->pool_dist[i] : FLT_MAX;
        const bool ok = id != kClean;
        const uint64_t m = ballot(ok);
        wave_sync();
        if (ok) {
            const uint32_t pos = n + prefix_count(m);
            pl->pool_id[pos] = id;
            pl->pool_dist[pos] = d;   // pos <= i and earlier chunks are already consumed
        }
        n += __popcll(m);
        wave_sync();
    }
    return n;
}

// stable compaction of the pool by the keep flags of entries [first, pool_size)
template <int MAX_BEAM, class PL>
__device__ __forceinline__ uint32_t compact_pool(PL* pl, uint32_t first, uint32_t pool_size, int lane) {
    uint32_t n = 0;
    for (uint32_t base = 0; base < pool_size; base += 64) {
        const uint32_t i = base + lane;
        const bool ok = i >= first && i < pool_size && pl->keep[i] != 0;
        const uint32_t id = i < pool_size ? pl->pool_id[i] : 0u;
        const float d = i < pool_size ? pl->pool_dist[i] : 0.f;
        const uint64_t m = ballot(ok);
        wave_sync();
        if (ok) {
            const uint32_t pos = n + prefix_count(m);
            pl->pool_id[pos] = id;
            pl->pool_dist[pos] = d;
        }
        n += __popcll(m);
        wave_sync();
    }
    return n;
}

// sync_prune: returns the neighbour count; pl->neighbor[0..round_up32(D)) holds ids (+segment_start) or invalid
template <int MAX_BEAM, int DIMV, class PL>
__device__ __forceinline__ uint32_t prune_pool(PL* pl, uint32_t pool_size, const float* data, uint32_t dim,
                                               uint32_t segment_start, uint32_t graph_degree, float relaxant, int metric,
                                               int lane, uint32_t& rows_scored) {
    for (uint32_t i = lane; i < PL::kCap; i += 64) pl->neighbor[i] = kInvalid;
    wave_sync();
    uint32_t nsize = 0;
    while (nsize < graph_degree && pool_size > 0) {
        const uint32_t head = pl->pool_id[0] + segment_start;
        if (lane == 0) pl->neighbor[nsize] = head;
        nsize++;
        RowRegs<DIMV> hrow;
        load_row<DIMV>(hrow, data + static_cast<size_t>(head) * dim, dim, RowShape<DIMV>::lane_in_row(lane));
        rows_scored += pool_size - 1;
        score_list<DIMV>(hrow, data, dim, metric, 1, pool_size, lane,
                         [pl, segment_start](uint32_t idx) { return pl->pool_id[idx] + segment_start; },
                         [pl, relaxant](uint32_t idx, float d) { pl->keep[idx] = (relaxant * d < pl->pool_dist[idx]) ? 0u : 1u; });
        wave_sync();
        pool_size = compact_pool<MAX_BEAM>(pl, 1, pool_size, lane);
    }
    return nsize;
}

// sync_prune_refine: heads must be valid, differ from `self` and not already be in the row (pl->s_graph)
template <int MAX_BEAM, int DIMV, class PL>
__device__ __forceinline__ uint32_t prune_pool_refine(PL* pl, uint32_t pool_size, const float* data, uint32_t dim,
                                                      uint32_t self, uint32_t graph_degree, uint32_t need, float relaxant,
                                                      int metric, int lane, uint32_t& rows_scored) {
    for (uint32_t i = lane; i < PL::kCap; i += 64) pl->neighbor[i] = kInvalid;
    wave_sync();
    uint32_t nsize = 0;
    while (nsize < need && pool_size > 0) {
        uint32_t position = kInvalid;  // select_point: first admissible pool entry
        for (uint32_t base = 0; base < pool_size && position == kInvalid; base += 64) {
            const uint32_t i = base + lane;
            bool ok = false;
            if (i < pool_size) {
                const uint32_t id = pl->pool_id[i];
                ok = id != kInvalid && id != self;
                for (uint32_t j = 0; ok && j < graph_degree; j++) ok = pl->s_graph[j] != id;
            }
            const uint64_t m = ballot(ok);
            if (m) position = base + __builtin_ctzll(m);
        }
        if (position == kInvalid) break;
        const uint32_t head = pl->pool_id[position];
        if (lane == 0) pl->neighbor[nsize] = head;
        nsize++;
        RowRegs<DIMV> hrow;
        load_row<DIMV>(hrow, data + static_cast<size_t>(head) * dim, dim, RowShape<DIMV>::lane_in_row(lane));
        rows_scored += pool_size - position;
        score_list<DIMV>(hrow, data, dim, metric, position, pool_size, lane,
                         [pl](uint32_t idx) { return pl->pool_id[idx]; },
                         [pl, relaxant](uint32_t idx, float d) { pl->keep[idx] = (relaxant * d < pl->pool_dist[idx]) ? 0u : 1u; });
        wave_sync();
        pool_size = compact_pool<MAX_BEAM>(pl, position, pool_size, lane);
    }
    return nsize;
}

// map_to_graph_boundary: merge the boundary copy's neighbours (reorder ids in pl->neighbor) into `row`
template <int MAX_BEAM, class PL>
__device__ __forceinline__ void merge_boundary_row(PL* pl, uint32_t* row, const uint32_t* map,
                                                   uint32_t graph_degree, int lane) {
    const uint32_t max_degree = round_up32(graph_degree);
    for (uint32_t i = lane; i < PL::kCap; i += 64) pl->s_graph[i] = i < graph_degree ? row[i] : kInvalid;
    if (lane < static_cast<int>(PL::kCap / 32)) pl->dup_mask[lane] = 0;
    wave_sync();
    uint32_t nfresh = 0, ndup = 0;
    for (uint32_t base = 0; base < max_degree; base += 64) {
        const uint32_t i = base + lane;
        const bool valid = i < graph_degree && pl->neighbor[i] != kInvalid;
        const uint32_t index = valid ? map[pl->neighbor[i]] : kInvalid;
        bool found = false;
        uint32_t j = 0;
        if (valid) {
            for (; j < graph_degree; j++) {
                const uint32_t g = pl->s_graph[j];
                if (g == kInvalid) break;
                if (g == index) { found = true; break; }
            }
        }
        const uint64_t mf = ballot(valid && !found), md = ballot(valid && found);
        if (valid && !found) pl->fresh[nfresh + prefix_count(mf)] = index;
        if (valid && found) atomicOr(&pl->dup_mask[j >> 5], 1u << (j & 31));
        nfresh += __popcll(mf);
        ndup += __popcll(md);
    }
    wave_sync();
    if (ndup >= graph_degree / 2) {  // fill empty slots front to back
        uint32_t used = 0;
        for (uint32_t base = 0; base < max_degree && used < nfresh; base += 64) {
            const uint32_t i = base + lane;
            const bool hole = i < graph_degree && pl->s_graph[i] == kInvalid;
            const uint64_t m = ballot(hole);
            const uint32_t pos = used + prefix_count(m);
            if (hole && pos < nfresh) row[i] = pl->fresh[pos];
            used += __popcll(m);
        }
    } else {  // overwrite from the tail: empty slots and entries the copy did not confirm
        const uint32_t max_need = graph_degree / 2 - ndup;
        const uint32_t need = nfresh < max_need ? nfresh : max_need;
        uint32_t used = 0;
        for (uint32_t base = 0; base < max_degree && used < need; base += 64) {
            const uint32_t i = base + lane;
            const uint32_t gi = max_degree - 1 - i;
            bool ok = false;
            if (i < max_degree && gi < graph_degree) {
                const bool dup = (pl->dup_mask[gi >> 5] >> (gi & 31)) & 1u;
                ok = pl->s_graph[gi] == kInvalid || !dup;
            }
            const uint64_t m = ballot(ok);
            const uint32_t pos = used + prefix_count(m);
            if (ok && pos < need) row[gi] = pl->fresh[pos];
            used += __popcll(m);
        }
    }
}

}  // namespace glide
