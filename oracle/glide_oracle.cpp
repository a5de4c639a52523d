// CPU oracle for the GLIDE build/search path.  TEST INFRASTRUCTURE ONLY -- see glide_oracle.h.
// Sequential (per item) restatement of the reference's kernels; OpenMP only across items.
#include "glide_oracle.h"

#include <algorithm>
#include <cfloat>
#include <cmath>
#include <cstring>
#include <numeric>
#include <queue>
#include <random>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

constexpr uint32_t kInvalid = 0xffffffffu;
constexpr uint32_t kExplored = 0x80000000u;  // utils.cuh:5-8
constexpr uint32_t kClean = 0x7fffffffu;

inline uint32_t round_up32(uint32_t p) { return (p + 31u) & ~31u; }  // utils.cuh:21-23
inline uint32_t swz(uint32_t x) { return x ^ (x >> 5); }             // utils.cuh:30-37 (X_MAX <= 1024)

int set_threads(int threads) {
#ifdef _OPENMP
    if (threads <= 0) threads = omp_get_max_threads();
    return threads;
#else
    (void) threads;
    return 1;
#endif
}

// ---------------------------------------------------------------- bitonic (bitonic.cuh:24-212)
// swap_if_needed, register form (bitonic.cuh:25-34): no exchange on equal keys.
inline void cmpx(float *k, uint32_t *v, uint32_t a, uint32_t b, bool asc) {
    if ((k[a] != k[b]) && ((k[a] < k[b]) != asc)) {
        std::swap(k[a], k[b]);
        std::swap(v[a], v[b]);
    }
}

// warp_merge_core<N> for power-of-two N (generic, N==2 and N==1 specialisations agree with it):
// bitonic.cuh:47-88,165-199.  Element e = N*lane + i.
void warp_merge(float *k, uint32_t *v, uint32_t N, uint32_t range) {
    if (range == 1) {
        for (uint32_t b = 2; b <= N; b <<= 1) {
            for (uint32_t c = b / 2; c >= 1; c >>= 1) {
                for (uint32_t lane = 0; lane < 32; lane++) {
                    for (uint32_t i = 0; i < N; i++) {
                        uint32_t j = i ^ c;
                        if (i >= j) continue;
                        uint32_t line_id = i + N * lane;
                        bool p = static_cast<bool>(line_id & b) == static_cast<bool>(line_id & c);
                        cmpx(k, v, N * lane + i, N * lane + j, p);
                    }
                }
            }
        }
        return;
    }
    const uint32_t b = range;
    for (uint32_t c = b / 2; c >= 1; c >>= 1) {
        // shuffle form (bitonic.cuh:36-44): each lane keeps its own or takes its partner's item.
        for (uint32_t lane = 0; lane < 32; lane++) {
            uint32_t other = lane ^ c;
            if (lane > other) continue;
            bool p_lo = static_cast<bool>(lane & b) == static_cast<bool>(lane & c);
            bool p_hi = static_cast<bool>(other & b) == static_cast<bool>(other & c);
            for (uint32_t i = 0; i < N; i++) {
                uint32_t e0 = N * lane + i, e1 = N * other + i;
                float k0 = k[e0], k1 = k[e1];
                uint32_t v0 = v[e0], v1 = v[e1];
                if ((k0 != k1) && ((k0 < k1) != p_lo)) { k[e0] = k1; v[e0] = v1; }
                if ((k1 != k0) && ((k1 < k0) != p_hi)) { k[e1] = k0; v[e1] = v0; }
            }
        }
    }
    for (uint32_t lane = 0; lane < 32; lane++) {
        bool p = ((lane & b) == 0);
        for (uint32_t c = N / 2; c >= 1; c >>= 1) {
            for (uint32_t i = 0; i < N; i++) {
                uint32_t j = i ^ c;
                if (i >= j) continue;
                cmpx(k, v, N * lane + i, N * lane + j, p);
            }
        }
    }
}

// the in-lane stage of the range>=2 branch iterates c outermost in the reference; lanes are independent
// so the per-lane loop nest above is equivalent.

void warp_sort(float *k, uint32_t *v, uint32_t N) {  // bitonic.cuh:207-212
    for (uint32_t range = 1; range <= 32; range <<= 1) warp_merge(k, v, N, range);
}

bool pow2(uint32_t x) { return x && !(x & (x - 1)); }

// ---------------------------------------------------------------- hashmap (hashmap.cuh:23-56)
inline void hash_init(uint32_t *table, uint32_t bitlen) {
    std::fill(table, table + (1u << bitlen), kInvalid);
}
inline uint32_t hash_insert(uint32_t *table, uint32_t bitlen, uint32_t key) {
    const uint32_t size = 1u << bitlen;
    const uint32_t mask = size - 1;
    uint32_t index = (key ^ (key >> bitlen)) & mask;
    for (uint32_t i = 0; i < size; i++) {
        uint32_t old = table[index];
        if (old == kInvalid) {
            table[index] = key;
            return 1;
        } else if (old == key) {
            return 0;
        }
        index = (index + 1) & mask;
    }
    return 0;
}

// ---------------------------------------------------------------- distance (distance.cuh:9-27)
inline float dist32(const float *a, const float *b, uint32_t dim, int metric) {
    float part[32];
    for (uint32_t l = 0; l < 32; l++) part[l] = 0.0f;
    uint32_t full = dim & ~31u;
    for (uint32_t base = 0; base < full; base += 32) {
        for (uint32_t l = 0; l < 32; l++) {
            float diff = a[base + l] - b[base + l];
            part[l] = fmaf(diff, diff, part[l]);
        }
    }
    for (uint32_t i = full; i < dim; i++) {
        float diff = a[i] - b[i];
        part[i - full] = fmaf(diff, diff, part[i - full]);
    }
    // shfl_down tree; lane 0 only needs lanes below `offset*2`
    for (uint32_t offset = 16; offset > 0; offset >>= 1)
        for (uint32_t l = 0; l < offset; l++) part[l] += part[l + offset];
    return metric == GO_METRIC_EUCLIDEAN ? sqrtf(part[0]) : part[0];
}

// ---------------------------------------------------------------- kernel_config.cuh buckets
uint32_t max_candidate(uint32_t degree) { return degree <= 64 ? 64 : degree <= 128 ? 128 : degree <= 256 ? 256 : 0; }
uint32_t max_beam(uint32_t beam) { return beam <= 64 ? 64 : beam <= 128 ? 128 : beam <= 256 ? 256 : beam <= 512 ? 512 : 0; }

// distance.cuh:29-60
void sort_with_key_value(uint32_t max_number, uint32_t number, uint32_t *vals, float *keys) {
    const uint32_t N = (max_number + 31) / 32;
    std::vector<float> k(32 * N);
    std::vector<uint32_t> v(32 * N);
    for (uint32_t lane = 0; lane < 32; lane++)
        for (uint32_t i = 0; i < N; i++) {
            uint32_t j = lane + 32 * i;
            k[N * lane + i] = j < number ? keys[j] : FLT_MAX;
            v[N * lane + i] = j < number ? vals[j] : kInvalid;
        }
    warp_sort(k.data(), v.data(), N);
    for (uint32_t j = 0; j < 32 * N; j++)
        if (j < number) {
            keys[j] = k[j];
            vals[j] = v[j];
        }
}

// search_kernel.cuh:9-37 (single-warp branch)
void sort_for_candidate_1(uint32_t max_cand, float *cd, uint32_t *ci, uint32_t degree, uint32_t beam) {
    const uint32_t N = max_cand / 32;
    float k[256];
    uint32_t v[256];
    for (uint32_t lane = 0; lane < 32; lane++)
        for (uint32_t i = 0; i < N; i++) {
            uint32_t j = lane + 32 * i;
            k[N * lane + i] = j < degree ? cd[j] : FLT_MAX;
            v[N * lane + i] = j < degree ? ci[j] : kInvalid;
        }
    warp_sort(k, v, N);
    for (uint32_t j = 0; j < 32 * N; j++)
        if (j < degree && j < beam) {
            cd[swz(j)] = k[j];
            ci[swz(j)] = v[j];
        }
}

// search_kernel.cuh:38-94 (two-warp branch, taken when MAX_CANDIDATE > 128: every launch has at least 64 threads).
// Each warp sorts its half of the slots; a half-cleaner across the halves leaves the smaller keys with warp 0 and the
// larger with warp 1; each warp then merges its half.  Sequential restatement of the data-parallel steps (no step
// reads a location another thread of the same step writes).
void sort_for_candidate_2(uint32_t max_cand, float *cd, uint32_t *ci, uint32_t degree, uint32_t beam) {
    const uint32_t per_warp = (max_cand + 1) / 2, N = (per_warp + 31) / 32;
    float key[2][256];
    uint32_t val[2][256];
    for (uint32_t w = 0; w < 2; w++) {
        for (uint32_t lane = 0; lane < 32; lane++)
            for (uint32_t i = 0; i < N; i++) {
                const uint32_t j = lane + 32 * i + per_warp * w;
                key[w][N * lane + i] = j < degree ? cd[j] : FLT_MAX;
                val[w][N * lane + i] = j < degree ? ci[j] : kInvalid;
            }
        warp_sort(key[w], val[w], N);
    }
    for (uint32_t w = 0; w < 2; w++)
        for (uint32_t jl = 0; jl < 32 * N; jl++) {
            const uint32_t j = jl + per_warp * w;
            if (j < degree && jl < beam) {
                cd[swz(j)] = key[w][jl];
                ci[swz(j)] = val[w][jl];
            }
        }
    const uint32_t warps_used = std::min<uint32_t>((beam + per_warp - 1) / per_warp, 2);
    for (uint32_t w = 0; w < warps_used; w++)
        for (uint32_t jl = 0; jl < 32 * N; jl++) {
            const uint32_t kl = per_warp - 1 - jl, j = jl + per_warp * w, k = max_cand - 1 - j;
            if (j >= degree || k >= degree || kl >= beam) continue;
            const float other = cd[swz(k)];
            if (key[w][jl] == other) continue;
            if ((w == 0) == (key[w][jl] > other)) {
                key[w][jl] = other;
                val[w][jl] = ci[swz(k)];
            }
        }
    for (uint32_t w = 0; w < warps_used; w++) warp_merge(key[w], val[w], N, 32);
    for (uint32_t w = 0; w < warps_used; w++)
        for (uint32_t jl = 0; jl < 32 * N; jl++) {
            const uint32_t j = jl + per_warp * w;
            if (j < degree && j < beam) {
                cd[swz(j)] = key[w][jl];
                ci[swz(j)] = val[w][jl];
            }
        }
}

void sort_for_candidate(uint32_t max_cand, float *cd, uint32_t *ci, uint32_t degree, uint32_t beam) {
    if (max_cand > 128) sort_for_candidate_2(max_cand, cd, ci, degree, beam);
    else sort_for_candidate_1(max_cand, cd, ci, degree, beam);
}

void sort_for_beam_1(uint32_t max_b, float *bd, uint32_t *bi, uint32_t beam, const float *cd, const uint32_t *ci, uint32_t degree,
                     bool first);

// search_kernel.cuh:149-232 (two-warp branch, taken when MAX_BEAM > 256).  In place on the beam buffer: candidates
// displace larger beam entries from the tail, the two halves are compare-exchanged element by element, the smallest
// touched index of each half ("turning point") is tracked, and each warp merges its half, laid out as
// [untouched prefix | padding | touched rest] over MAX_BEAM / 2 slots.
void sort_for_beam_2(uint32_t max_b, float *bd, uint32_t *bi, uint32_t beam, const float *cd, const uint32_t *ci, uint32_t degree,
                     bool first) {
    if (first) {
        sort_for_beam_1(max_b, bd, bi, beam, cd, ci, degree, true);
        return;
    }
    const uint32_t per_warp = (max_b + 1) / 2, N = (per_warp + 31) / 32, half = beam / 2;
    uint32_t ws[3] = {half, half, half};
    for (uint32_t k = 0; k < std::min(degree, beam); k++) {
        const uint32_t j = beam - 1 - k;
        if (bd[swz(j)] > cd[swz(k)]) {
            bd[swz(j)] = cd[swz(k)];
            bi[swz(j)] = ci[swz(k)];
            if (j < half) ws[2] = std::min(ws[2], j);
            else ws[1] = std::min(ws[1], j - half);
        }
    }
    for (uint32_t j = 0; j < half; j++) {
        const uint32_t k = j + half;
        if (bd[swz(j)] > bd[swz(k)]) {
            std::swap(bd[swz(j)], bd[swz(k)]);
            std::swap(bi[swz(j)], bi[swz(k)]);
            ws[0] = std::min(ws[0], j);
        }
    }
    if (ws[2] < half) ws[1] = ws[2];
    float key[2][256];
    uint32_t val[2][256];
    for (uint32_t w = 0; w < 2; w++) {
        const uint32_t turning = ws[w];
        for (uint32_t slot = 0; slot < 32 * N; slot++) {
            uint32_t k = beam, j = slot;
            if (j < turning) {
                k = j + half * w;
            } else if (j >= max_b / 2 - half) {
                j -= max_b / 2 - half;
                if (turning <= j && j < half) k = j + half * w;
            }
            key[w][slot] = k < beam ? bd[swz(k)] : FLT_MAX;
            val[w][slot] = k < beam ? bi[swz(k)] : kInvalid;
        }
    }
    for (uint32_t w = 0; w < 2; w++) {
        warp_merge(key[w], val[w], N, 32);
        for (uint32_t j = 0; j < 32 * N; j++)
            if (j < half) {
                bd[swz(j + half * w)] = key[w][j];
                bi[swz(j + half * w)] = val[w][j];
            }
    }
}

void sort_for_beam(uint32_t max_b, float *bd, uint32_t *bi, uint32_t beam, const float *cd, const uint32_t *ci, uint32_t degree,
                   bool first) {
    if (max_b > 256) sort_for_beam_2(max_b, bd, bi, beam, cd, ci, degree, first);
    else sort_for_beam_1(max_b, bd, bi, beam, cd, ci, degree, first);
}

// search_kernel.cuh:97-148 (single-warp branch)
void sort_for_beam_1(uint32_t max_b, float *bd, uint32_t *bi, uint32_t beam, const float *cd, const uint32_t *ci,
                     uint32_t degree, bool first) {
    if (first) {
        for (uint32_t i = 0; i < beam; i++) {
            bd[swz(i)] = i < degree ? cd[swz(i)] : FLT_MAX;
            bi[swz(i)] = i < degree ? ci[swz(i)] : kInvalid;
        }
        return;
    }
    const uint32_t N = max_b / 32;
    float k[512];
    uint32_t v[512];
    for (uint32_t j = 0; j < 32 * N; j++) {
        k[j] = j < beam ? bd[swz(j)] : FLT_MAX;
        v[j] = j < beam ? bi[swz(j)] : kInvalid;
    }
    for (uint32_t j = 0; j < 32 * N; j++) {
        uint32_t kk = max_b - 1 - j;
        if (kk >= beam || kk >= degree) continue;
        float ck = cd[swz(kk)];
        if (k[j] > ck) {
            k[j] = ck;
            v[j] = ci[swz(kk)];
        }
    }
    warp_merge(k, v, N, 32);
    for (uint32_t j = 0; j < 32 * N; j++)
        if (j < beam) {
            bd[swz(j)] = k[j];
            bi[swz(j)] = v[j];
        }
}

// ---------------------------------------------------------------- beam-search core
struct SearchCfg {
    uint32_t beam, degree, max_iter, min_iter, hash_bit, reset;
    uint32_t max_cand, max_b;
    int metric;
};

struct Scratch {
    std::vector<uint32_t> ids;
    std::vector<float> dists;
    std::vector<uint32_t> hash;
    std::vector<uint32_t> neighbor, s_graph, bitmap;
    std::vector<uint32_t> cent_ids;
    std::vector<float> cent_dists;
    go_stats st{0, 0, 0};
    void prepare(const SearchCfg &c, uint32_t graph_degree_out, uint32_t centroid_num) {
        uint32_t rb = round_up32(c.beam + c.degree);
        ids.assign(rb, kInvalid);
        dists.assign(rb, FLT_MAX);
        hash.resize(1u << c.hash_bit);
        neighbor.assign(round_up32(graph_degree_out) + 32, kInvalid);
        s_graph.assign(round_up32(graph_degree_out) + 32, kInvalid);
        bitmap.assign((c.beam + 31) / 32 + 1, 0);
        cent_ids.resize(std::max<uint32_t>(centroid_num, 1));
        cent_dists.resize(std::max<uint32_t>(centroid_num, 1));
    }
};

// search_kernel.cuh:292-325
bool select_current_point(uint32_t *beam_ids, uint32_t beam, uint32_t &select) {
    select = kInvalid;
    for (uint32_t j = 0; j < beam; j++) {
        uint32_t jj = swz(j);
        if ((beam_ids[jj] & kExplored) == 0) {
            select = beam_ids[jj];
            beam_ids[jj] |= kExplored;
            return true;
        }
    }
    return false;
}

// search_kernel.cuh:362-391 (also get_init :336-360 when `init_exclude` differs and parent is a start point)
void expand(const SearchCfg &c, Scratch &s, const float *query, const float *data, uint32_t dim,
            const uint32_t *graph, uint32_t parent, uint32_t exclude_insert, uint32_t exclude_score) {
    uint32_t *ci = s.ids.data() + c.beam;
    float *cd = s.dists.data() + c.beam;
    if (parent != kInvalid) s.st.graph_rows++;
    for (uint32_t i = 0; i < c.degree; i++) {
        uint32_t nid = kInvalid;
        if (parent != kInvalid) nid = graph[static_cast<size_t>(parent) * c.degree + i];
        uint32_t flag = (nid != kInvalid && nid != exclude_insert) ? hash_insert(s.hash.data(), c.hash_bit, nid) : 0;
        ci[i] = flag == 1 ? nid : kInvalid;
    }
    for (uint32_t i = 0; i < c.degree; i++) {
        uint32_t idx = ci[i];
        if (idx != kInvalid && idx != exclude_score) {
            cd[i] = dist32(query, data + static_cast<size_t>(idx) * dim, dim, c.metric);
            s.st.rows_scored++;
        } else {
            cd[i] = FLT_MAX;
        }
    }
}

// main loop shared by search_kernel.cuh:433-482 and get_neighbors graph_kernel.cuh:16-63.
void beam_loop(const SearchCfg &c, Scratch &s, const float *query, const float *data, uint32_t dim,
               const uint32_t *graph, uint32_t point_id) {
    uint32_t *bi = s.ids.data();
    float *bd = s.dists.data();
    uint32_t *ci = bi + c.beam;
    float *cd = bd + c.beam;
    uint32_t iter = 0;
    bool terminate = false;
    while (true) {
        sort_for_candidate(c.max_cand, cd, ci, c.degree, c.beam);
        sort_for_beam(c.max_b, bd, bi, c.beam, cd, ci, c.degree, iter == 0);
        s.st.iterations++;
        bool reset = ((iter + 1) % c.reset == 0);
        if (reset) hash_init(s.hash.data(), c.hash_bit);
        if (iter + 1 == c.max_iter) break;
        uint32_t select;
        if (!select_current_point(bi, c.beam, select)) terminate = true;
        if (reset) {  // hashmap_restore search_kernel.cuh:327-334 (raw index order; includes 0x7fffffff for empty slots)
            for (uint32_t i = 0; i < c.beam; i++) hash_insert(s.hash.data(), c.hash_bit, bi[i] & kClean);
        }
        if (terminate && iter >= c.min_iter) break;
        expand(c, s, query, data, dim, graph, select, point_id, kInvalid);
        iter++;
    }
}

// search_kernel.cuh:248-290
void result_init(const SearchCfg &c, Scratch &s, const float *query, const float *data, uint32_t dim,
                 const uint32_t *graph, const uint32_t *start_points, const float *centroids,
                 uint32_t centroid_num, uint32_t max_centroid) {
    for (uint32_t i = 0; i < centroid_num; i++) {
        s.cent_ids[i] = i;
        s.cent_dists[i] = dist32(query, centroids + static_cast<size_t>(i) * dim, dim, c.metric);
    }
    sort_with_key_value(max_centroid, centroid_num, s.cent_ids.data(), s.cent_dists.data());
    uint32_t node = start_points[s.cent_ids[0]];
    expand(c, s, query, data, dim, graph, node, kInvalid, kInvalid);
}

uint32_t max_centroid_search(uint32_t centroid_num, uint32_t graph_degree) {  // kernel_config.cuh:161-171
    if (centroid_num <= 32) return 32;
    if (graph_degree <= 64) return 64;
    if (graph_degree <= 128) return 128;
    return 256;
}

bool make_cfg(SearchCfg &c, uint32_t beam, uint32_t degree, uint32_t max_iter, uint32_t min_iter, uint32_t hash_bit,
              uint32_t reset, int metric) {
    c.beam = beam;
    c.degree = degree;
    c.max_iter = max_iter;
    c.min_iter = min_iter;
    c.hash_bit = hash_bit;
    c.reset = reset ? reset : 1;
    c.metric = metric;
    c.max_cand = max_candidate(degree);
    c.max_b = max_beam(beam);
    if (c.max_cand == 0 || c.max_b == 0) return false;
    if (beam == 0 || degree == 0 || hash_bit > 20) return false;
    return true;
}

// graph_kernel.cuh:65-67: strip the explored bit; then drop slots that never held a node.
// (The reference would dereference id 0x7fffffff in the prune; the guard is a stable compaction.)
uint32_t clean_and_compact(const SearchCfg &c, Scratch &s) {
    uint32_t *bi = s.ids.data();
    float *bd = s.dists.data();
    uint32_t n = 0;
    std::vector<uint32_t> ti(c.beam);
    std::vector<float> td(c.beam);
    for (uint32_t i = 0; i < c.beam; i++) {
        uint32_t id = bi[swz(i)] & kClean;
        if (id != kClean) {
            ti[n] = id;
            td[n] = bd[swz(i)];
            n++;
        }
    }
    for (uint32_t i = 0; i < c.beam; i++) {
        bi[swz(i)] = i < n ? ti[i] : kClean;
        bd[swz(i)] = i < n ? td[i] : FLT_MAX;
    }
    return n;
}

// graph_kernel.cuh:70-143
uint32_t sync_prune(const float *data, uint32_t dim, uint32_t segment_start, uint32_t *bi, float *bd,
                    uint32_t pool_size, uint32_t graph_degree, float relaxant, int metric, uint32_t *neighbor,
                    go_stats *st) {
    uint32_t nsize = 0;
    std::vector<uint32_t> keep;
    while (nsize < graph_degree && pool_size > 0) {
        uint32_t id = bi[swz(0)] + segment_start;
        neighbor[nsize++] = id;
        keep.clear();
        for (uint32_t i = 1; i < pool_size; i++) {
            uint32_t index = bi[swz(i)] + segment_start;
            float d = dist32(data + static_cast<size_t>(id) * dim, data + static_cast<size_t>(index) * dim, dim, metric);
            if (st) st->rows_scored++;
            bool allow = !(relaxant * d < bd[swz(i)]);
            if (allow) keep.push_back(i);
        }
        for (uint32_t t = 0; t < keep.size(); t++) {
            uint32_t src = keep[t];
            uint32_t id_t = bi[swz(src)];
            float d_t = bd[swz(src)];
            bi[swz(t)] = id_t;
            bd[swz(t)] = d_t;
        }
        pool_size = static_cast<uint32_t>(keep.size());
    }
    return nsize;
}

// graph_kernel.cuh:455-578
uint32_t sync_prune_refine(const float *data, uint32_t dim, uint32_t point_id, uint32_t *bi, float *bd,
                           uint32_t pool_size, uint32_t graph_degree, uint32_t need_num, const uint32_t *s_graph,
                           float relaxant, int metric, uint32_t *neighbor, go_stats *st) {
    uint32_t nsize = 0;
    std::vector<uint32_t> keep;
    while (nsize < need_num && pool_size > 0) {
        uint32_t position = kInvalid;
        for (uint32_t i = 0; i < pool_size; i++) {  // select_point
            uint32_t id = bi[swz(i)];
            if (id == kInvalid || id == point_id) continue;
            bool exist = false;
            for (uint32_t j = 0; j < graph_degree; j++)
                if (s_graph[j] == id) { exist = true; break; }
            if (!exist) { position = i; break; }
        }
        if (position == kInvalid) break;
        uint32_t id = bi[swz(position)];
        neighbor[nsize++] = id;
        keep.clear();
        for (uint32_t i = position; i < pool_size; i++) {
            uint32_t index = bi[swz(i)];
            float d = dist32(data + static_cast<size_t>(id) * dim, data + static_cast<size_t>(index) * dim, dim, metric);
            if (st) st->rows_scored++;
            bool allow = !(relaxant * d < bd[swz(i)]);
            if (allow) keep.push_back(i);
        }
        for (uint32_t t = 0; t < keep.size(); t++) {
            uint32_t src = keep[t];
            uint32_t id_t = bi[swz(src)];
            float d_t = bd[swz(src)];
            bi[swz(t)] = id_t;
            bd[swz(t)] = d_t;
        }
        pool_size = static_cast<uint32_t>(keep.size());
    }
    return nsize;
}

// graph_kernel.cuh:160-247
void merge_boundary_row(uint32_t *row, uint32_t D, const uint32_t *neighbor_in, const uint32_t *map) {
    const uint32_t maxD = round_up32(D);
    std::vector<uint32_t> s_graph(maxD, kInvalid), fresh;
    std::vector<uint8_t> dup(maxD, 0);
    for (uint32_t i = 0; i < D; i++) s_graph[i] = row[i];
    uint32_t repetitive = 0;
    for (uint32_t i = 0; i < D; i++) {
        if (neighbor_in[i] == kInvalid) continue;
        uint32_t index = map[neighbor_in[i]];
        bool found = false;
        uint32_t j;
        for (j = 0; j < D; j++) {
            if (s_graph[j] == kInvalid) break;
            if (s_graph[j] == index) { found = true; break; }
        }
        if (found) {
            dup[j] = 1;
            repetitive++;
        } else {
            fresh.push_back(index);
        }
    }
    uint32_t valid = static_cast<uint32_t>(fresh.size());
    if (repetitive >= D / 2) {
        uint32_t t = 0;
        for (uint32_t i = 0; i < D && t < valid; i++)
            if (s_graph[i] == kInvalid) row[i] = fresh[t++];
    } else {
        uint32_t max_need = D / 2 - repetitive;
        uint32_t need = valid < max_need ? valid : max_need;
        uint32_t t = 0;
        for (uint32_t i = 0; i < maxD && t < need; i++) {
            uint32_t gi = maxD - 1 - i;
            if (gi >= D) continue;
            bool invalid = s_graph[gi] == kInvalid;
            if (invalid || !dup[gi]) row[gi] = fresh[t++];
        }
    }
}

}  // namespace

// =================================================================================== C API
extern "C" {

uint32_t go_hash_bitlen(uint32_t beam, uint32_t graph_degree, float fill, uint32_t min_bitlen_in) {  // params.cuh:49-66
    uint32_t max_visited = beam + graph_degree;
    uint32_t min_bitlen = 8, max_bitlen = 13;
    if (min_bitlen < min_bitlen_in) min_bitlen = min_bitlen_in;
    uint32_t bitlen = min_bitlen;
    while (max_visited > (1u << bitlen) * fill) bitlen += 1;
    if (bitlen > max_bitlen) bitlen = max_bitlen;
    return bitlen;
}

uint32_t go_hash_reset_interval(uint32_t beam, uint32_t graph_degree, float fill, uint32_t bitlen) {  // params.cuh:68-80
    uint32_t interval = 1;
    while (1) {
        const auto max_visited = beam + graph_degree * (interval + 1);
        if (max_visited > (1u << bitlen) * fill) break;
        interval += 1;
    }
    return interval;
}

void go_adjust_search_params(uint32_t min_iterations, uint32_t *max_iterations, uint32_t *beam) {  // params.cuh:82-99
    uint32_t mi = *max_iterations;
    if (*max_iterations == 0) mi = 1 + std::min(*beam * 1.1, *beam + 10.0);
    if (*max_iterations < min_iterations) mi = min_iterations;
    if (*max_iterations < mi) *max_iterations = mi;
    if (*beam % 32) *beam += 32 - (*beam % 32);
}

uint32_t go_nnd_extended_degree(uint32_t degree) {  // nn_descent.cuh:1427-1428
    return round_up32(static_cast<uint32_t>(degree * (degree <= 32 ? 1.0 : 1.3)));
}

uint32_t go_xorshift32(uint32_t u) {  // utils.cuh:14-19
    u ^= u >> 13;
    u ^= u << 27;
    u ^= u >> 5;
    return u * 0x9E3779B9u;
}

int go_bitonic_warp_sort(float *keys, uint32_t *vals, uint32_t M) {
    if (M % 32 || !pow2(M / 32)) return -1;
    warp_sort(keys, vals, M / 32);
    return 0;
}

int go_bitonic_warp_merge(float *keys, uint32_t *vals, uint32_t M, uint32_t range) {
    if (M % 32 || !pow2(M / 32) || !pow2(range) || range > 32) return -1;
    warp_merge(keys, vals, M / 32, range);
    return 0;
}

int go_sort_with_key_value(uint32_t max_number, uint32_t number, uint32_t *vals, float *keys) {
    if (max_number % 32 || !pow2(max_number / 32)) return -1;
    sort_with_key_value(max_number, number, vals, keys);
    return 0;
}

int go_sort_for_candidate(uint32_t max_cand, float *cd, uint32_t *ci, uint32_t degree, uint32_t beam) {
    if (max_cand % 32 || !pow2(max_cand / 32) || max_cand > 256) return -1;
    sort_for_candidate(max_cand, cd, ci, degree, beam);
    return 0;
}

int go_sort_for_beam(uint32_t max_b, float *bd, uint32_t *bi, uint32_t beam, const float *cd, const uint32_t *ci,
                     uint32_t degree, int first) {
    if (max_b % 32 || !pow2(max_b / 32) || max_b > 512) return -1;
    sort_for_beam(max_b, bd, bi, beam, cd, ci, degree, first != 0);
    return 0;
}

void go_hashmap_init(uint32_t *table, uint32_t bitlen) { hash_init(table, bitlen); }

void go_hashmap_insert_seq(uint32_t *table, uint32_t bitlen, const uint32_t *keys, uint32_t n, uint32_t *flags) {
    for (uint32_t i = 0; i < n; i++) flags[i] = hash_insert(table, bitlen, keys[i]);
}

float go_distance(const float *a, const float *b, uint32_t dim, int metric) { return dist32(a, b, dim, metric); }

uint32_t go_max_candidate(uint32_t degree) { return max_candidate(degree); }
uint32_t go_max_beam(uint32_t beam) { return max_beam(beam); }
uint32_t go_max_centroid_search(uint32_t c, uint32_t d) { return max_centroid_search(c, d); }
uint32_t go_max_centroid_partition(uint32_t c) { return c <= 32 ? 32 : c <= 64 ? 64 : c <= 128 ? 128 : c <= 256 ? 256 : 0; }

static void add_stats(go_stats *dst, const go_stats &src) {
    if (!dst) return;
#pragma omp critical(go_stats_add)
    {
        dst->iterations += src.iterations;
        dst->rows_scored += src.rows_scored;
        dst->graph_rows += src.graph_rows;
    }
}

int go_search(const float *data, uint32_t num, uint32_t dim, const uint32_t *graph, uint32_t graph_degree,
              const float *centroids, uint32_t centroid_num, const uint32_t *start_points, const float *queries,
              uint32_t query_num, uint32_t top_k, uint32_t beam, uint32_t max_iterations, uint32_t min_iterations,
              uint32_t hash_bit, uint32_t hash_reset_interval, int metric, uint32_t *result_ids,
              float *result_dists, go_stats *stats, int threads) {
    (void) num;
    SearchCfg c;
    if (!make_cfg(c, beam, graph_degree, max_iterations, min_iterations, hash_bit, hash_reset_interval, metric))
        return -1;
    if (top_k > beam) return -1;
    const uint32_t maxc = max_centroid_search(centroid_num, graph_degree);
    if (stats) *stats = go_stats{0, 0, 0};
    threads = set_threads(threads);
#pragma omp parallel num_threads(threads)
    {
        Scratch s;
#pragma omp for schedule(dynamic, 16)
        for (int64_t q = 0; q < static_cast<int64_t>(query_num); q++) {
            s.prepare(c, graph_degree, centroid_num);
            const float *query = queries + static_cast<size_t>(q) * dim;
            hash_init(s.hash.data(), c.hash_bit);
            result_init(c, s, query, data, dim, graph, start_points, centroids, centroid_num, maxc);
            beam_loop(c, s, query, data, dim, graph, kInvalid);
            for (uint32_t i = 0; i < top_k; i++) {  // search_kernel.cuh:484-489
                result_dists[static_cast<size_t>(q) * top_k + i] = s.dists[swz(i)];
                result_ids[static_cast<size_t>(q) * top_k + i] = s.ids[swz(i)] & kClean;
            }
        }
        add_stats(stats, s.st);
    }
    return 0;
}

int go_partition_assign(const float *data, uint32_t num, uint32_t dim, const float *centroids, uint32_t centroid_num,
                        float boundary_factor, int metric, uint32_t *segment_indexes, uint32_t *segment_lengths,
                        float *nearest_dists, int threads) {
    const uint32_t maxc = go_max_centroid_partition(centroid_num);
    if (maxc == 0 || centroid_num == 0) return -1;
    threads = set_threads(threads);
    std::vector<uint8_t> is_boundary(num);
#pragma omp parallel num_threads(threads)
    {
        std::vector<uint32_t> ids(centroid_num);
        std::vector<float> dists(centroid_num);
#pragma omp for schedule(static)
        for (int64_t p = 0; p < static_cast<int64_t>(num); p++) {
            for (uint32_t i = 0; i < centroid_num; i++) {
                ids[i] = i;
                dists[i] = dist32(data + static_cast<size_t>(p) * dim, centroids + static_cast<size_t>(i) * dim, dim, metric);
            }
            sort_with_key_value(maxc, centroid_num, ids.data(), dists.data());
            segment_indexes[p * 3] = ids[0];
            is_boundary[p] = (centroid_num > 1 && dists[1] / dists[0] <= boundary_factor) ? 1 : 0;
            if (nearest_dists) {
                nearest_dists[p * 2] = dists[0];
                nearest_dists[p * 2 + 1] = centroid_num > 1 ? dists[1] : FLT_MAX;
            }
        }
    }
    // slot ids: the reference takes them from atomicAdd (arbitrary order); here in point order.
    for (uint32_t i = 0; i <= centroid_num; i++) segment_lengths[i] = 0;
    for (uint32_t p = 0; p < num; p++) {
        segment_indexes[p * 3 + 1] = segment_lengths[segment_indexes[p * 3]]++;
        segment_indexes[p * 3 + 2] = is_boundary[p] ? segment_lengths[centroid_num]++ : kInvalid;
    }
    return 0;
}

void go_reorder(const float *data, uint32_t num, uint32_t dim, const uint32_t *segment_indexes,
                const uint32_t *segment_starts, float *reorder_data, uint32_t *map) {
    for (uint32_t p = 0; p < num; p++) {
        uint32_t rid = segment_starts[segment_indexes[p * 3]] + segment_indexes[p * 3 + 1];
        std::memcpy(reorder_data + static_cast<size_t>(rid) * dim, data + static_cast<size_t>(p) * dim, dim * sizeof(float));
        map[rid] = p;
        uint32_t b = segment_indexes[p * 3 + 2];
        if (b != kInvalid) {
            uint32_t bid = num + b;
            std::memcpy(reorder_data + static_cast<size_t>(bid) * dim, data + static_cast<size_t>(p) * dim, dim * sizeof(float));
            map[bid] = p;
        }
    }
}

int go_build_subgraph(const float *reorder_data, uint32_t num, uint32_t dim, const uint32_t *knn_graph,
                      uint32_t knn_degree, const uint32_t *map, const uint32_t *segment_starts,
                      const uint32_t *segment_lengths, uint32_t segment_num, const uint32_t *start_points,
                      uint32_t graph_degree, uint32_t beam, uint32_t max_iterations, uint32_t min_iterations,
                      uint32_t hash_bit, uint32_t hash_reset_interval, float relaxant, int metric, uint32_t *graph,
                      go_stats *stats, int threads) {
    SearchCfg c;
    if (!make_cfg(c, beam, knn_degree, max_iterations, min_iterations, hash_bit, hash_reset_interval, metric)) return -1;
    if (stats) *stats = go_stats{0, 0, 0};
    threads = set_threads(threads);
#pragma omp parallel num_threads(threads)
    {
        Scratch s;
#pragma omp for schedule(dynamic, 64)
        for (int64_t pp = 0; pp < static_cast<int64_t>(num); pp++) {
            uint32_t p = static_cast<uint32_t>(pp);
            uint32_t seg;
            for (seg = 0; seg < segment_num; seg++)
                if (p < segment_starts[seg] + segment_lengths[seg]) break;
            const uint32_t seg_start = segment_starts[seg];
            const float *sdata = reorder_data + static_cast<size_t>(seg_start) * dim;
            const uint32_t *sgraph = knn_graph + static_cast<size_t>(seg_start) * knn_degree;
            const float *point = reorder_data + static_cast<size_t>(p) * dim;
            s.prepare(c, graph_degree, 0);
            hash_init(s.hash.data(), c.hash_bit);
            // get_init (search_kernel.cuh:336-360): every neighbour is hashed; the one equal to the *global* id is not scored
            expand(c, s, point, sdata, dim, sgraph, start_points[seg], kInvalid, p);
            beam_loop(c, s, point, sdata, dim, sgraph, p - seg_start);
            uint32_t pool = clean_and_compact(c, s);
            std::fill(s.neighbor.begin(), s.neighbor.end(), kInvalid);
            sync_prune(reorder_data, dim, seg_start, s.ids.data(), s.dists.data(), pool, graph_degree, relaxant,
                       metric, s.neighbor.data(), &s.st);
            uint32_t *row = graph + static_cast<size_t>(map[p]) * graph_degree;  // map_to_graph_sub graph_kernel.cuh:152-158
            for (uint32_t i = 0; i < graph_degree; i++)
                row[i] = s.neighbor[i] == kInvalid ? kInvalid : map[s.neighbor[i]];
        }
        add_stats(stats, s.st);
    }
    return 0;
}

int go_build_boundary(const float *reorder_data, uint32_t num, uint32_t reorder_num, uint32_t dim,
                      const uint32_t *knn_graph, uint32_t knn_degree, const uint32_t *map, uint32_t start_point,
                      uint32_t graph_degree, uint32_t beam, uint32_t max_iterations, uint32_t min_iterations,
                      uint32_t hash_bit, uint32_t hash_reset_interval, float relaxant, int metric, uint32_t *graph,
                      go_stats *stats, int threads) {
    SearchCfg c;
    if (!make_cfg(c, beam, knn_degree, max_iterations, min_iterations, hash_bit, hash_reset_interval, metric)) return -1;
    if (stats) *stats = go_stats{0, 0, 0};
    threads = set_threads(threads);
    const uint32_t seg_start = num;
    const float *sdata = reorder_data + static_cast<size_t>(seg_start) * dim;
    const uint32_t *sgraph = knn_graph + static_cast<size_t>(seg_start) * knn_degree;
#pragma omp parallel num_threads(threads)
    {
        Scratch s;
#pragma omp for schedule(dynamic, 64)
        for (int64_t pp = num; pp < static_cast<int64_t>(reorder_num); pp++) {
            uint32_t p = static_cast<uint32_t>(pp);
            const float *point = reorder_data + static_cast<size_t>(p) * dim;
            s.prepare(c, graph_degree, 0);
            hash_init(s.hash.data(), c.hash_bit);
            expand(c, s, point, sdata, dim, sgraph, start_point, kInvalid, p);
            beam_loop(c, s, point, sdata, dim, sgraph, p - seg_start);
            uint32_t pool = clean_and_compact(c, s);
            std::fill(s.neighbor.begin(), s.neighbor.end(), kInvalid);
            sync_prune(reorder_data, dim, seg_start, s.ids.data(), s.dists.data(), pool, graph_degree, relaxant,
                       metric, s.neighbor.data(), &s.st);
            merge_boundary_row(graph + static_cast<size_t>(map[p]) * graph_degree, graph_degree, s.neighbor.data(), map);
        }
        add_stats(stats, s.st);
    }
    return 0;
}

void go_merge_boundary_row(uint32_t *row, uint32_t graph_degree, const uint32_t *neighbors, const uint32_t *map) {
    merge_boundary_row(row, graph_degree, neighbors, map);
}

uint32_t go_prune(const float *data, uint32_t dim, uint32_t segment_start, uint32_t *pool_ids, float *pool_dists,
                  uint32_t pool_size, uint32_t graph_degree, float relaxant, int metric, uint32_t *neighbors) {
    // explicit pool in plain order -> swizzled scratch
    uint32_t padded = round_up32(pool_size) + 32;
    std::vector<uint32_t> bi(padded, kClean);
    std::vector<float> bd(padded, FLT_MAX);
    for (uint32_t i = 0; i < pool_size; i++) {
        bi[swz(i)] = pool_ids[i];
        bd[swz(i)] = pool_dists[i];
    }
    for (uint32_t i = 0; i < round_up32(graph_degree); i++) neighbors[i] = kInvalid;
    return sync_prune(data, dim, segment_start, bi.data(), bd.data(), pool_size, graph_degree, relaxant, metric,
                      neighbors, nullptr);
}

void go_reverse_edges(uint32_t *graph, uint32_t num, uint32_t D) {
    std::vector<uint32_t> rev(static_cast<size_t>(num) * D, kInvalid), cnt(num, 0);
    for (uint32_t c = 0; c < D; c++) {
        for (uint32_t s = 0; s < num; s++) {
            uint32_t t = graph[static_cast<size_t>(s) * D + c];
            if (t >= num) continue;
            bool have = false;
            for (uint32_t i = 0; i < D; i++)
                if (graph[static_cast<size_t>(t) * D + i] == s) { have = true; break; }
            if (have) continue;
            uint32_t pos = cnt[t]++;
            if (pos < D) rev[static_cast<size_t>(t) * D + pos] = s;
        }
    }
    for (uint32_t p = 0; p < num; p++) {  // insert_reverse_kernel graph_kernel.cuh:416-453
        uint32_t nrev = cnt[p] > D ? D : cnt[p];
        uint32_t t = 0;
        for (uint32_t i = 0; i < D && t < nrev; i++)
            if (graph[static_cast<size_t>(p) * D + i] == kInvalid) graph[static_cast<size_t>(p) * D + i] = rev[static_cast<size_t>(p) * D + t++];
    }
}

int go_refine(const float *data, uint32_t num, uint32_t dim, uint32_t *graph, uint32_t graph_degree,
              const float *centroids, uint32_t centroid_num, const uint32_t *start_points, uint32_t beam,
              uint32_t max_iterations, uint32_t min_iterations, uint32_t hash_bit, uint32_t hash_reset_interval,
              float relaxant, int metric, go_stats *stats, int threads) {
    SearchCfg c;
    if (!make_cfg(c, beam, graph_degree, max_iterations, min_iterations, hash_bit, hash_reset_interval, metric)) return -1;
    const uint32_t maxc = max_centroid_search(centroid_num, graph_degree);
    if (stats) *stats = go_stats{0, 0, 0};
    threads = set_threads(threads);
    // The reference refines in place while other blocks still read the rows (a race); here every
    // search reads the graph as it was before refinement.
    std::vector<uint32_t> snap(graph, graph + static_cast<size_t>(num) * graph_degree);
#pragma omp parallel num_threads(threads)
    {
        Scratch s;
#pragma omp for schedule(dynamic, 64)
        for (int64_t pp = 0; pp < static_cast<int64_t>(num); pp++) {
            uint32_t p = static_cast<uint32_t>(pp);
            const uint32_t *srow = snap.data() + static_cast<size_t>(p) * graph_degree;
            uint32_t need = 0;
            for (uint32_t i = 0; i < graph_degree; i++) need += srow[i] == kInvalid;
            if (need == 0) continue;
            const float *point = data + static_cast<size_t>(p) * dim;
            s.prepare(c, graph_degree, centroid_num);
            for (uint32_t i = 0; i < graph_degree; i++) s.s_graph[i] = srow[i];
            hash_init(s.hash.data(), c.hash_bit);
            result_init(c, s, point, data, dim, snap.data(), start_points, centroids, centroid_num, maxc);
            beam_loop(c, s, point, data, dim, snap.data(), p);
            uint32_t pool = clean_and_compact(c, s);
            std::fill(s.neighbor.begin(), s.neighbor.end(), kInvalid);
            sync_prune_refine(data, dim, p, s.ids.data(), s.dists.data(), pool, graph_degree, need, s.s_graph.data(),
                              relaxant, metric, s.neighbor.data(), &s.st);
            uint32_t t = 0;
            uint32_t *row = graph + static_cast<size_t>(p) * graph_degree;
            for (uint32_t i = 0; i < graph_degree; i++)
                if (srow[i] == kInvalid) row[i] = s.neighbor[t++];
        }
        add_stats(stats, s.st);
    }
    return 0;
}

// ----------------------------------------------------------------------------- large path
// select_segment_kernel search_kernel.cuh:546-607.  The reference resets only the first row of the output and leaves
// the others uninitialised; every row starts at 0xffffffff here (what the consumer search_kernel.cuh:676-686 expects).
int go_select_segments(const float *queries, uint32_t query_num, uint32_t dim, const float *centroids,
                       uint32_t centroid_num, uint32_t min_segment_num, float boundary_factor, int metric,
                       uint32_t *segment_ids) {
    const uint32_t maxc = go_max_centroid_partition(centroid_num);   // kernel_config.cuh:290-304
    if (maxc == 0) return -1;
    std::vector<uint32_t> ids(centroid_num);
    std::vector<float> dists(centroid_num);
    for (uint32_t q = 0; q < query_num; q++) {
        uint32_t *out = segment_ids + static_cast<size_t>(q) * centroid_num;
        for (uint32_t i = 0; i < centroid_num; i++) {
            out[i] = kInvalid;
            ids[i] = i;
            dists[i] = dist32(queries + static_cast<size_t>(q) * dim, centroids + static_cast<size_t>(i) * dim, dim, metric);
        }
        sort_with_key_value(maxc, centroid_num, ids.data(), dists.data());
        uint32_t allow_num = 0;
        for (uint32_t i = 0; i < centroid_num; i++) {
            if (dists[i] / dists[0] <= boundary_factor) {
                out[i] = ids[i];
                allow_num++;
            }
        }
        if (allow_num < min_segment_num) {
            uint32_t need = min_segment_num - allow_num;
            for (uint32_t i = 0; i < need && allow_num + i < centroid_num; i++) out[allow_num + i] = ids[allow_num + i];
        }
    }
    return 0;
}

// search_on_sub_kernel + result_merge search_kernel.cuh:609-765 for one segment; final_* are updated in place
int go_search_sub(const float *seg_data, uint32_t dim, const uint32_t *seg_graph, uint32_t graph_degree, const uint32_t *seg_map,
                  const float *queries, uint32_t query_num, const uint32_t *segment_ids, uint32_t centroid_num,
                  uint32_t segment_id, uint32_t start_point, uint32_t top_k, uint32_t beam, uint32_t max_iterations,
                  uint32_t min_iterations, uint32_t hash_bit, uint32_t hash_reset_interval, int metric,
                  uint32_t *final_ids, float *final_dists, go_stats *stats, int threads) {
    SearchCfg c;
    if (!make_cfg(c, beam, graph_degree, max_iterations, min_iterations, hash_bit, hash_reset_interval, metric)) return -1;
    const uint32_t max_topk = top_k <= 32 ? 32 : top_k <= 64 ? 64 : top_k <= 128 ? 128 : 0;   // kernel_config.cuh:312-323
    if (max_topk == 0 || top_k > beam) return -1;
    if (stats) *stats = go_stats{0, 0, 0};
    threads = set_threads(threads);
#pragma omp parallel num_threads(threads)
    {
        Scratch s;
#pragma omp for schedule(dynamic, 16)
        for (int64_t q = 0; q < static_cast<int64_t>(query_num); q++) {
            bool is_search = false;
            for (uint32_t i = 0; i < centroid_num; i++) {
                uint32_t v = segment_ids[static_cast<size_t>(q) * centroid_num + i];
                if (v == segment_id) { is_search = true; break; }
                if (v == kInvalid) break;
            }
            if (!is_search) continue;
            const float *query = queries + static_cast<size_t>(q) * dim;
            s.prepare(c, graph_degree, 0);
            hash_init(s.hash.data(), c.hash_bit);
            expand(c, s, query, seg_data, dim, seg_graph, start_point, kInvalid, kInvalid);   // get_init with point_id = max
            beam_loop(c, s, query, seg_data, dim, seg_graph, kInvalid);
            // result_merge: half-cleaner against the reversed beam head, then the final merge network
            const uint32_t N = max_topk / 32;
            float k[128];
            uint32_t v[128];
            float *fd = final_dists + static_cast<size_t>(q) * top_k;
            uint32_t *fi = final_ids + static_cast<size_t>(q) * top_k;
            for (uint32_t j = 0; j < max_topk; j++) {
                k[j] = j < top_k ? fd[j] : FLT_MAX;
                v[j] = j < top_k ? fi[j] : kInvalid;
            }
            for (uint32_t j = 0; j < max_topk; j++) {
                uint32_t kk = max_topk - 1 - j;
                if (kk >= top_k) continue;
                float rk = s.dists[swz(kk)];
                if (k[j] > rk) {
                    k[j] = rk;
                    v[j] = seg_map[s.ids[swz(kk)] & kClean];
                }
            }
            warp_merge(k, v, N, 32);
            for (uint32_t j = 0; j < top_k; j++) {
                fd[j] = k[j];
                fi[j] = v[j];
            }
        }
        add_stats(stats, s.st);
    }
    return 0;
}

// build_for_large_kernel graph_kernel.cuh:675-728: one staged segment, local ids in and out
int go_build_segment(const float *seg_data, uint32_t num, uint32_t dim, const uint32_t *knn_graph, uint32_t knn_degree,
                     uint32_t start_point, uint32_t graph_degree, uint32_t beam, uint32_t max_iterations,
                     uint32_t min_iterations, uint32_t hash_bit, uint32_t hash_reset_interval, float relaxant, int metric,
                     uint32_t *graph, go_stats *stats, int threads) {
    SearchCfg c;
    if (!make_cfg(c, beam, knn_degree, max_iterations, min_iterations, hash_bit, hash_reset_interval, metric)) return -1;
    if (stats) *stats = go_stats{0, 0, 0};
    threads = set_threads(threads);
#pragma omp parallel num_threads(threads)
    {
        Scratch s;
#pragma omp for schedule(dynamic, 64)
        for (int64_t pp = 0; pp < static_cast<int64_t>(num); pp++) {
            uint32_t p = static_cast<uint32_t>(pp);
            const float *point = seg_data + static_cast<size_t>(p) * dim;
            s.prepare(c, graph_degree, 0);
            hash_init(s.hash.data(), c.hash_bit);
            expand(c, s, point, seg_data, dim, knn_graph, start_point, kInvalid, p);
            beam_loop(c, s, point, seg_data, dim, knn_graph, p);
            uint32_t pool = clean_and_compact(c, s);
            std::fill(s.neighbor.begin(), s.neighbor.end(), kInvalid);
            sync_prune(seg_data, dim, 0, s.ids.data(), s.dists.data(), pool, graph_degree, relaxant, metric, s.neighbor.data(), &s.st);
            for (uint32_t i = 0; i < graph_degree; i++) graph[static_cast<size_t>(p) * graph_degree + i] = s.neighbor[i];   // map_to_graph :145-150
        }
        add_stats(stats, s.st);
    }
    return 0;
}

// refine_for_large_kernel graph_kernel.cuh:730-821 (entry = the segment's start point), snapshot semantics as go_refine
int go_refine_segment(const float *seg_data, uint32_t num, uint32_t dim, uint32_t *graph, uint32_t graph_degree,
                      uint32_t start_point, uint32_t beam, uint32_t max_iterations, uint32_t min_iterations, uint32_t hash_bit,
                      uint32_t hash_reset_interval, float relaxant, int metric, go_stats *stats, int threads) {
    SearchCfg c;
    if (!make_cfg(c, beam, graph_degree, max_iterations, min_iterations, hash_bit, hash_reset_interval, metric)) return -1;
    if (stats) *stats = go_stats{0, 0, 0};
    threads = set_threads(threads);
    std::vector<uint32_t> snap(graph, graph + static_cast<size_t>(num) * graph_degree);
#pragma omp parallel num_threads(threads)
    {
        Scratch s;
#pragma omp for schedule(dynamic, 64)
        for (int64_t pp = 0; pp < static_cast<int64_t>(num); pp++) {
            uint32_t p = static_cast<uint32_t>(pp);
            const uint32_t *srow = snap.data() + static_cast<size_t>(p) * graph_degree;
            uint32_t need = 0;
            for (uint32_t i = 0; i < graph_degree; i++) need += srow[i] == kInvalid;
            if (need == 0) continue;
            const float *point = seg_data + static_cast<size_t>(p) * dim;
            s.prepare(c, graph_degree, 0);
            for (uint32_t i = 0; i < graph_degree; i++) s.s_graph[i] = srow[i];
            hash_init(s.hash.data(), c.hash_bit);
            expand(c, s, point, seg_data, dim, snap.data(), start_point, kInvalid, p);
            beam_loop(c, s, point, seg_data, dim, snap.data(), p);
            uint32_t pool = clean_and_compact(c, s);
            std::fill(s.neighbor.begin(), s.neighbor.end(), kInvalid);
            sync_prune_refine(seg_data, dim, p, s.ids.data(), s.dists.data(), pool, graph_degree, need, s.s_graph.data(), relaxant,
                              metric, s.neighbor.data(), &s.st);
            uint32_t t = 0;
            uint32_t *row = graph + static_cast<size_t>(p) * graph_degree;
            for (uint32_t i = 0; i < graph_degree; i++)
                if (srow[i] == kInvalid) row[i] = s.neighbor[t++];
        }
        add_stats(stats, s.st);
    }
    return 0;
}

// ----------------------------------------------------------------------------- brute force + kmeans
void go_bruteforce_knn(const float *data, uint32_t num, uint32_t dim, const float *queries, uint32_t query_num,
                       uint32_t k, int metric, int exclude_self, uint32_t *ids, float *dists, int threads) {
    threads = set_threads(threads);
#pragma omp parallel for num_threads(threads) schedule(dynamic, 4)
    for (int64_t q = 0; q < static_cast<int64_t>(query_num); q++) {
        const float *qv = queries + static_cast<size_t>(q) * dim;
        std::priority_queue<std::pair<float, uint32_t>> heap;  // max-heap on (dist, id)
        for (uint32_t i = 0; i < num; i++) {
            if (exclude_self && i == static_cast<uint32_t>(q)) continue;
            const float *dv = data + static_cast<size_t>(i) * dim;
            float acc = 0.0f;
            for (uint32_t t = 0; t < dim; t++) {
                float diff = qv[t] - dv[t];
                acc += diff * diff;
            }
            if (heap.size() < k) {
                heap.emplace(acc, i);
            } else if (std::make_pair(acc, i) < heap.top()) {
                heap.pop();
                heap.emplace(acc, i);
            }
        }
        uint32_t n = static_cast<uint32_t>(heap.size());
        for (uint32_t i = n; i < k; i++) {
            ids[static_cast<size_t>(q) * k + i] = kInvalid;
            dists[static_cast<size_t>(q) * k + i] = FLT_MAX;
        }
        while (!heap.empty()) {
            n--;
            ids[static_cast<size_t>(q) * k + n] = heap.top().second;
            float d = heap.top().first;
            dists[static_cast<size_t>(q) * k + n] = metric == GO_METRIC_EUCLIDEAN ? sqrtf(d) : d;
            heap.pop();
        }
    }
}

// Greedy k-means++ seeding as the HIP library's glide_hip_kmeans_seed does it (no counterpart in the reference tree:
// the reference calls cuvs::cluster::kmeans::fit, whose default initialisation is of the k-means++ family).  Every
// step draws 2 + floor(ln k) candidate rows with probability min_dist[i] / sum (the sum taken over 1024 chunks in
// double; draw j of step s is a hash of (seed, 16 s + j)) and keeps the candidate that leaves the smallest potential
// sum_i min(min_dist[i], |x_i - candidate|^2), the first one on a tie.
static uint32_t seed_hash(uint32_t seed, uint32_t step) {
    uint32_t x = seed * 0x9E3779B9u + step * 0x85EBCA6Bu + 0x6A09E667u;
    x ^= x >> 16; x *= 0x7FEB352Du; x ^= x >> 15; x *= 0x846CA68Bu; x ^= x >> 16;
    return x;
}
static uint32_t kmeans_trials(uint32_t k) {
    uint32_t t = 2;
    for (uint32_t v = k; v >= 3; v = static_cast<uint32_t>(v / 2.718281828459045)) t++;   // 2 + floor(ln k) for k >= 1
    return t > 8 ? 8 : t;
}
// first index whose running sum of the positive entries exceeds target; the last positive entry if none does
static uint32_t locate(const double *v, uint32_t len, double target, double *before) {
    double run = 0.0;
    uint32_t last = 0;
    for (uint32_t i = 0; i < len; i++) {
        if (v[i] > 0.0) {
            last = i;
            if (run + v[i] > target) { *before = run; return i; }
        }
        run += v[i];
    }
    double r = 0.0;
    for (uint32_t i = 0; i < last; i++) r += v[i];
    *before = r;
    return last;
}

void go_kmeans_seed(const float *sample, uint32_t n, uint32_t dim, uint32_t k, uint32_t seed, float *centroids,
                    uint32_t *chosen_out) {
    std::vector<float> min_dist(n, FLT_MAX);
    const uint32_t chunk = (n + 1023) / 1024, trials = kmeans_trials(k);
    auto dist_to = [&](uint32_t row, uint32_t i) {
        float acc = 0.0f;
        for (uint32_t t = 0; t < dim; t++) {
            const float diff = sample[static_cast<size_t>(i) * dim + t] - sample[static_cast<size_t>(row) * dim + t];
            acc += diff * diff;
        }
        return acc;
    };
    for (uint32_t step = 0; step < k; step++) {
        uint32_t chosen = seed_hash(seed, 16 * step) % n;
        if (step > 0) {
            std::vector<double> part(1024, 0.0);
            double total = 0.0;
            for (uint32_t t = 0; t < 1024; t++) {
                const uint64_t lo = std::min<uint64_t>(static_cast<uint64_t>(t) * chunk, n), hi = std::min<uint64_t>(lo + chunk, n);
                for (uint64_t i = lo; i < hi; i++) part[t] += static_cast<double>(min_dist[i]);
            }
            for (uint32_t t = 0; t < 1024; t++) total += part[t];
            if (total > 0.0) {
                double best_pot = 0.0;
                for (uint32_t j = 0; j < trials; j++) {
                    const uint32_t h = seed_hash(seed, 16 * step + j);
                    const double target = static_cast<double>(h >> 8) * (1.0 / 16777216.0) * total;
                    double before = 0.0;
                    const uint32_t c = locate(part.data(), 1024, target, &before);
                    const uint32_t base = c * chunk, len = static_cast<uint32_t>(std::min<uint64_t>(static_cast<uint64_t>(base) + chunk, n) - base);
                    std::vector<double> seg(len);
                    for (uint32_t i = 0; i < len; i++) seg[i] = static_cast<double>(min_dist[base + i]);
                    double b2 = 0.0;
                    const uint32_t cand = base + locate(seg.data(), len, target - before, &b2);
                    double pot = 0.0;
                    for (uint32_t i = 0; i < n; i++) pot += static_cast<double>(std::min(min_dist[i], dist_to(cand, i)));
                    if (j == 0 || pot < best_pot) { best_pot = pot; chosen = cand; }
                }
            }
        }
        if (chosen_out) chosen_out[step] = chosen;
        std::memcpy(centroids + static_cast<size_t>(step) * dim, sample + static_cast<size_t>(chosen) * dim, dim * sizeof(float));
        for (uint32_t i = 0; i < n; i++) {
            const float d = dist_to(chosen, i);
            min_dist[i] = step == 0 ? d : std::min(min_dist[i], d);
        }
    }
}

// Lloyd steps from the centroids passed in (init != 0) or from k rows of a shuffle of the sample (init == 0)
void go_kmeans_from(const float *sample, uint32_t n, uint32_t dim, uint32_t k, uint32_t iterations, float *centroids);

void go_kmeans(const float *sample, uint32_t n, uint32_t dim, uint32_t k, uint32_t iterations, uint32_t seed,
               float *centroids) {
    std::mt19937 gen(seed);
    std::vector<uint32_t> perm(n);
    std::iota(perm.begin(), perm.end(), 0u);
    std::shuffle(perm.begin(), perm.end(), gen);
    for (uint32_t c = 0; c < k; c++)
        std::memcpy(centroids + static_cast<size_t>(c) * dim, sample + static_cast<size_t>(perm[c % n]) * dim, dim * sizeof(float));
    go_kmeans_from(sample, n, dim, k, iterations, centroids);
}

void go_kmeans_from(const float *sample, uint32_t n, uint32_t dim, uint32_t k, uint32_t iterations, float *centroids) {
    std::vector<double> sums(static_cast<size_t>(k) * dim);
    std::vector<uint32_t> counts(k);
    for (uint32_t it = 0; it < iterations; it++) {
        std::fill(sums.begin(), sums.end(), 0.0);
        std::fill(counts.begin(), counts.end(), 0u);
        for (uint32_t p = 0; p < n; p++) {
            float best = FLT_MAX;
            uint32_t bc = 0;
            for (uint32_t c = 0; c < k; c++) {
                float acc = 0.0f;
                for (uint32_t t = 0; t < dim; t++) {
                    float diff = sample[static_cast<size_t>(p) * dim + t] - centroids[static_cast<size_t>(c) * dim + t];
                    acc += diff * diff;
                }
                if (acc < best) { best = acc; bc = c; }
            }
            counts[bc]++;
            for (uint32_t t = 0; t < dim; t++) sums[static_cast<size_t>(bc) * dim + t] += sample[static_cast<size_t>(p) * dim + t];
        }
        for (uint32_t c = 0; c < k; c++)
            if (counts[c])
                for (uint32_t t = 0; t < dim; t++)
                    centroids[static_cast<size_t>(c) * dim + t] = static_cast<float>(sums[static_cast<size_t>(c) * dim + t] / counts[c]);
    }
}

}  // extern "C"
