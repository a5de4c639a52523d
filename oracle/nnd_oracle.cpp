// CPU oracle, NN-descent part.  TEST INFRASTRUCTURE ONLY -- see glide_oracle.h.
//
// Restates the reference's per-partition NN-descent (nn_descent.cuh) as the *intended* algorithm:
// every partition is updated in every iteration until max_iterations or until its own update counter falls below the
// termination limit (go_nnd_build_ex; go_nnd_build runs the fixed count).  The reference's
// own host loop stops updating partitions >= 1 after two rounds (it passes a length where an end is
// expected, nn_descent.cuh:1276-1279 vs :1129-1135).  go_nnd_build_shipped restates that loop as it is written, so
// that what the shipped executable would score can be quoted next to the intended algorithm; nothing is compared
// against it.  Bit-level parity is unpinned (the reference is unseeded and racy); tests check graph recall.
#include "glide_oracle.h"

#include <algorithm>
#include <atomic>
#include <cfloat>
#include <climits>
#include <cmath>
#include <cstring>
#include <numeric>
#include <random>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

constexpr uint32_t kSeg = 32;          // SEGMENT_SIZE / DEGREE_ON_DEVICE  nn_descent.cuh:46-47
constexpr uint32_t kSamples = 32;      // NUM_SAMPLES                      nn_descent.cuh:391
constexpr uint32_t kBi = 64;           // MAX_NUM_BI_SAMPLES               nn_descent.cuh:392

inline uint32_t round_up32(uint32_t p) { return (p + 31u) & ~31u; }

// fp32 -> fp16 -> fp32 (round to nearest even), as preprocess_data_kernel stores halfs (nn_descent.cuh:445-488)
float round_half(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    uint32_t sign = x & 0x80000000u;
    uint32_t ax = x & 0x7fffffffu;
    float r;
    if (ax >= 0x47800000u) {  // >= 65536 -> inf (or nan)
        uint32_t y = sign | 0x7f800000u;
        std::memcpy(&r, &y, 4);
        return r;
    }
    if (ax < 0x38800000u) {  // subnormal half: quantum 2^-24
        float a = std::fabs(f);
        float q = std::nearbyintf(a * 16777216.0f) / 16777216.0f;
        return sign ? -q : q;
    }
    uint32_t rem = ax & 0x1fffu;
    ax &= ~0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (ax & 0x2000u))) ax += 0x2000u;
    if (ax >= 0x47800000u) ax = 0x7f800000u;
    uint32_t y = sign | ax;
    std::memcpy(&r, &y, 4);
    return r;
}

// ids carry an "old" flag in the sign bit (InternalID_t nn_descent.cuh:53-83)
inline int id_of(int v) { return v >= 0 ? v : -v - 1; }
inline bool is_new(int v) { return v >= 0; }
inline int mark_old(int v) { return v >= 0 ? -v - 1 : v; }

struct Bloom {  // nn_descent.cuh:203-276
    uint32_t sets;
    std::vector<bool> bits;
    static constexpr uint32_t kBits = 512;
    Bloom(uint32_t nrow, uint32_t sets_) : sets(sets_), bits(static_cast<size_t>(nrow) * kBits * sets_) {}
    static uint32_t h0(uint32_t v) { v *= 1103515245u; v += 12345u; v ^= v << 13; v ^= v >> 17; v ^= v << 5; return v; }
    static uint32_t h1(uint32_t v) { v *= 1664525u; v += 1013904223u; v ^= v << 13; v ^= v >> 17; v ^= v << 5; return v; }
    bool check_add(uint32_t row, uint32_t key) {  // true if already present; adds otherwise
        size_t base = (static_cast<size_t>(row) * sets + key % sets) * kBits;
        uint32_t h = h0(key);
        uint32_t idx[3];
        idx[0] = h % kBits;
        h += h1(key);
        idx[1] = h % kBits;
        h += h1(key);
        idx[2] = h % kBits;
        bool present = bits[base + idx[0]] && bits[base + idx[1]] && bits[base + idx[2]];
        if (present) return true;
        bits[base + idx[0]] = bits[base + idx[1]] = bits[base + idx[2]] = true;
        return false;
    }
};

// insert_to_ordered_list nn_descent.cuh:916-943
uint32_t insert_ordered(int *list, float *dl, uint32_t width, int nid, float dist) {
    if (dist > dl[width - 1]) return width;
    uint32_t pos = width;
    bool found = false;
    for (uint32_t i = 0; i < width; i++) {
        if (id_of(list[i]) == id_of(nid)) return width;
        if (!found && dl[i] > dist) { pos = i; found = true; }
    }
    if (pos == width) return pos;
    std::memmove(list + pos + 1, list + pos, sizeof(int) * (width - pos - 1));
    std::memmove(dl + pos + 1, dl + pos, sizeof(float) * (width - pos - 1));
    list[pos] = nid;
    dl[pos] = dist;
    return pos;
}

struct Partition {
    uint32_t n, dim, W, num_sub;
    const float *data;              // fp16-rounded rows, n x dim
    std::vector<float> norms;
    std::vector<int> lists;         // n x W, sub-lists of 32 keyed by id % num_sub
    std::vector<float> ldists;
    std::vector<int> dev_ids;       // n x 32 "device" result lists
    std::vector<float> dev_dists;
    std::vector<int> fwd_new, fwd_old, rev_new, rev_old;   // n x 32
    std::vector<uint32_t> n_fwd_new, n_fwd_old, n_rev_new, n_rev_old;
    std::vector<omp_lock_t> locks;
};

// insert_to_global_graph nn_descent.cuh:509-579 on the 32-wide device list
void dev_insert(Partition &P, uint32_t list_id, int elem_id, float elem_dist) {
    if (static_cast<uint32_t>(elem_id) == list_id) return;
    omp_set_lock(&P.locks[list_id]);
    int *ids = P.dev_ids.data() + static_cast<size_t>(list_id) * kSeg;
    float *ds = P.dev_dists.data() + static_cast<size_t>(list_id) * kSeg;
    // ResultItem ordering (nn_descent.cuh:107-131): '<' is lexicographic on (dist, id), '==' compares ids only,
    // '>' is !('==' or '<').  Lane l holds list[l]; lane 0's predecessor is {INT_MIN, FLT_MIN} (:551-553).
    auto lt = [](float d0, int i0, float d1, int i1) { return d0 == d1 ? i0 < i1 : d0 < d1; };
    int pos = -1;
    for (uint32_t l = 0; l < kSeg; l++) {
        float pd = l == 0 ? FLT_MIN : ds[l - 1];
        int pi = l == 0 ? INT_MAX : id_of(ids[l - 1]);
        float cd = ds[l];
        int ci = id_of(ids[l]);
        bool gt_prev = !(elem_id == pi) && !lt(elem_dist, elem_id, pd, pi);
        if (gt_prev && lt(elem_dist, elem_id, cd, ci)) { pos = static_cast<int>(l); break; }
    }
    if (pos >= 0) {
        std::memmove(ids + pos + 1, ids + pos, sizeof(int) * (kSeg - pos - 1));
        std::memmove(ds + pos + 1, ds + pos, sizeof(float) * (kSeg - pos - 1));
        ids[pos] = elem_id;  // new flag
        ds[pos] = elem_dist;
    }
    omp_unset_lock(&P.locks[list_id]);
}

// sample_graph / sample_segment_graph nn_descent.cuh:1040-1104
void sample_lists(Partition &P, bool sample_new) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < static_cast<int64_t>(P.n); i++) {
        uint32_t no = 0, nn = 0;
        int *list = P.lists.data() + static_cast<size_t>(i) * P.W;
        int *lo = P.fwd_old.data() + static_cast<size_t>(i) * kSamples;
        int *ln = P.fwd_new.data() + static_cast<size_t>(i) * kSamples;
        bool done = false;
        for (uint32_t j = 0; j < kSeg && !done; j++) {
            for (uint32_t k = 0; k < P.num_sub; k++) {
                int nb = list[k * kSeg + j];
                if (static_cast<uint32_t>(id_of(nb)) >= P.n) continue;
                if (!is_new(nb)) {
                    if (no < kSamples) lo[no++] = id_of(nb);
                } else if (sample_new) {
                    if (nn < kSamples) {
                        list[k * kSeg + j] = mark_old(nb);
                        ln[nn++] = id_of(nb);
                    }
                }
                if (no == kSamples && nn == kSamples) { done = true; break; }
            }
        }
        P.n_fwd_old[i] = no;
        if (sample_new) P.n_fwd_new[i] = nn;
    }
}

// add_rev_edges_kernel nn_descent.cuh:490-507, serialised in list order
void reverse_lists(uint32_t n, const std::vector<int> &fwd, const std::vector<uint32_t> &nf, std::vector<int> &rev,
                   std::vector<uint32_t> &nr) {
    std::fill(nr.begin(), nr.end(), 0u);
    for (uint32_t u = 0; u < n; u++)
        for (uint32_t j = 0; j < nf[u]; j++) {
            uint32_t v = static_cast<uint32_t>(fwd[static_cast<size_t>(u) * kSamples + j]);
            if (nr[v] < kSamples) rev[static_cast<size_t>(v) * kSamples + nr[v]++] = static_cast<int>(u);
        }
}

// local_join_kernel nn_descent.cuh:668-914 for one list
void local_join(Partition &P, uint32_t L, std::vector<float> &xn, std::vector<float> &xo, std::vector<float> &D) {
    int nl[kBi], ol[kBi];
    uint32_t nn = 0, no = 0;
    auto gather = [&](const std::vector<int> &fwd, uint32_t nf, const std::vector<int> &rev, uint32_t nr, int *out) {
        uint32_t c = 0;
        for (uint32_t i = 0; i < nf; i++) out[c++] = fwd[static_cast<size_t>(L) * kSamples + i];
        for (uint32_t i = 0; i < nr; i++) {  // remove_duplicates :625-666 (reverse entries already among the forward ones)
            int v = rev[static_cast<size_t>(L) * kSamples + i];
            bool dup = false;
            for (uint32_t j = 0; j < nf; j++) if (out[j] == v) { dup = true; break; }
            if (!dup) out[c++] = v;
        }
        return c;
    };
    nn = gather(P.fwd_new, P.n_fwd_new[L], P.rev_new, P.n_rev_new[L], nl);
    no = gather(P.fwd_old, P.n_fwd_old[L], P.rev_old, P.n_rev_old[L], ol);
    if (!nn) return;
    const uint32_t dim = P.dim;
    for (uint32_t i = 0; i < nn; i++) std::memcpy(&xn[static_cast<size_t>(i) * dim], P.data + static_cast<size_t>(nl[i]) * dim, dim * 4);
    for (uint32_t i = 0; i < no; i++) std::memcpy(&xo[static_cast<size_t>(i) * dim], P.data + static_cast<size_t>(ol[i]) * dim, dim * 4);
    auto tile = [&](const float *A, const int *ai, uint32_t na, const float *B, const int *bi, uint32_t nb) {
        for (uint32_t a = 0; a < na; a++)
            for (uint32_t b = 0; b < nb; b++) {
                const float *x = A + static_cast<size_t>(a) * dim, *y = B + static_cast<size_t>(b) * dim;
                float acc = 0.0f;
                for (uint32_t t = 0; t < dim; t++) acc += x[t] * y[t];
                D[a * kBi + b] = P.norms[ai[a]] + P.norms[bi[b]] - 2.0f * acc;
            }
    };
    // new x new
    tile(xn.data(), nl, nn, xn.data(), nl, nn);
    for (uint32_t a = 0; a < nn; a++) {  // get_min_item :581-623 (row)
        float best = FLT_MAX;
        int bid = -1;
        for (uint32_t b = 0; b < nn; b++)
            if (nl[b] != nl[a] && D[a * kBi + b] < best) { best = D[a * kBi + b]; bid = nl[b]; }
        if (bid >= 0 && static_cast<uint32_t>(bid) < P.n) dev_insert(P, static_cast<uint32_t>(nl[a]), bid, best);
    }
    if (!no) return;
    tile(xn.data(), nl, nn, xo.data(), ol, no);
    for (uint32_t a = 0; a < nn; a++) {
        float best = FLT_MAX;
        int bid = -1;
        for (uint32_t b = 0; b < no; b++)
            if (ol[b] != nl[a] && D[a * kBi + b] < best) { best = D[a * kBi + b]; bid = ol[b]; }
        if (bid >= 0 && static_cast<uint32_t>(bid) < P.n) dev_insert(P, static_cast<uint32_t>(nl[a]), bid, best);
    }
    for (uint32_t b = 0; b < no; b++) {  // column-wise
        float best = FLT_MAX;
        int bid = -1;
        for (uint32_t a = 0; a < nn; a++)
            if (nl[a] != ol[b] && D[a * kBi + b] < best) { best = D[a * kBi + b]; bid = nl[a]; }
        if (bid >= 0 && static_cast<uint32_t>(bid) < P.n) dev_insert(P, static_cast<uint32_t>(ol[b]), bid, best);
    }
}

// update_graph nn_descent.cuh:1106-1126; returns the update counter: insertions on rows whose index in the whole
// build (row_index_base + i) is a multiple of counter_interval = 100 (:1123)
// `rows` limits the update to local rows [0, rows); `as_shipped` compares the (partition-local) neighbour id with the row's
// index in the whole build, as update_graph :1117 / update_segment_graph :1139 do, instead of with its local index.
int64_t update_lists(Partition &P, const std::vector<int> &src_ids, const std::vector<float> &src_dists, uint32_t row_index_base,
                     uint32_t rows = 0xffffffffu, bool as_shipped = false) {
    int64_t counter = 0;
    const int64_t end = std::min<int64_t>(P.n, rows);
#pragma omp parallel for schedule(static) reduction(+ : counter)
    for (int64_t i = 0; i < end; i++) {
        for (uint32_t j = 0; j < kSeg; j++) {
            int nid = src_ids[static_cast<size_t>(i) * kSeg + j];
            float d = src_dists[static_cast<size_t>(i) * kSeg + j];
            if (d == FLT_MAX) break;
            if (static_cast<uint32_t>(id_of(nid)) == (as_shipped ? row_index_base + static_cast<uint32_t>(i) : static_cast<uint32_t>(i))) continue;
            uint32_t sub = static_cast<uint32_t>(id_of(nid)) % P.num_sub;
            uint32_t pos = insert_ordered(P.lists.data() + static_cast<size_t>(i) * P.W + sub * kSeg,
                                          P.ldists.data() + static_cast<size_t>(i) * P.W + sub * kSeg, kSeg, nid, d);
            if ((row_index_base + static_cast<uint32_t>(i)) % 100u == 0 && pos != kSeg) counter++;
        }
    }
    return counter;
}

// shipped != nullptr: the host loop as the reference ships it (GNND::build, nn_descent.cuh:1289-1402).
struct Shipped {
    uint32_t break_iteration;   // the iteration after whose joins every partition was marked converged (loop :1344-1351); iterations if never
    uint32_t last_join;         // out: the iteration of this partition's last join
};
void build_partition(const float *data, const float *norms_in, uint32_t n, uint32_t dim, uint32_t K, uint32_t iterations, uint32_t seed,
                     int32_t *out /* n x K local ids */, uint32_t row_index_base, float termination_limit, Shipped *shipped = nullptr,
                     const int32_t *start_lists = nullptr /* n x W local ids, sub-list after sub-list, replacing the shuffled lists */) {
    Partition P;
    P.n = n;
    P.dim = dim;
    P.data = data;
    P.W = go_nnd_extended_degree(K);
    P.num_sub = P.W / kSeg;
    uint32_t inter = static_cast<uint32_t>(1.5 * K);                 // params.cuh:23-24
    uint32_t ext_inter = go_nnd_extended_degree(inter);
    P.norms.assign(norms_in, norms_in + n);
    P.lists.assign(static_cast<size_t>(n) * P.W, INT_MAX);
    P.ldists.assign(static_cast<size_t>(n) * P.W, FLT_MAX);
    P.dev_ids.assign(static_cast<size_t>(n) * kSeg, INT_MAX);
    P.dev_dists.assign(static_cast<size_t>(n) * kSeg, FLT_MAX);
    for (auto *v : {&P.fwd_new, &P.fwd_old, &P.rev_new, &P.rev_old}) v->assign(static_cast<size_t>(n) * kSamples, 0);
    for (auto *v : {&P.n_fwd_new, &P.n_fwd_old, &P.n_rev_new, &P.n_rev_old}) v->assign(n, 0u);
    P.locks.resize(n);
    for (auto &l : P.locks) omp_init_lock(&l);
    Bloom bloom(n, ext_inter / kSeg);

    // init_random_graph nn_descent.cuh:1003-1038 (local ids); a caller that brings its own start lists (a test that wants
    // both sides of a comparison to start from the same random graph) replaces the shuffle, nothing else
    if (start_lists) {
        for (size_t i = 0; i < static_cast<size_t>(n) * P.W; i++)
            P.lists[i] = (start_lists[i] >= 0 && static_cast<uint32_t>(start_lists[i]) < n) ? start_lists[i] : INT_MAX;
    }
    for (uint32_t sub = 0; sub < P.num_sub && !start_lists; sub++) {
        uint32_t m = std::max<uint32_t>(n / P.num_sub, 1);
        std::vector<int> seq(m);
        std::iota(seq.begin(), seq.end(), 0);
        std::default_random_engine gen(sub + seed * 7919u);
        std::shuffle(seq.begin(), seq.end(), gen);
        for (uint32_t i = 0; i < n; i++) {
            uint32_t base = i * P.W + sub * kSeg;
            for (uint32_t j = 0; j < kSeg; j++) {
                uint32_t idx = base + j;
                int id = seq[idx % m] * static_cast<int>(P.num_sub) + static_cast<int>(sub);
                if (static_cast<uint32_t>(id) == i) id = seq[(idx + kSeg) % m] * static_cast<int>(P.num_sub) + static_cast<int>(sub);
                P.lists[static_cast<size_t>(i) * P.W + sub * kSeg + j] = id;
            }
        }
    }
    sample_lists(P, true);

    // Iteration structure of GNND::build (nn_descent.cuh:1289-1368): the join of iteration `it` runs on the device
    // while the host merges the results of iteration it-1 and resamples the old lists used by iteration it+1.
    std::vector<int> host_ids(static_cast<size_t>(n) * kSeg, INT_MAX), cur_old(static_cast<size_t>(n) * kSamples);
    std::vector<float> host_dists(static_cast<size_t>(n) * kSeg, FLT_MAX);
    std::vector<uint32_t> n_cur_old(n);
    // Termination (update_and_sample :1270-1284, loop :1305-1308): when the counter of a merge falls below the limit the
    // partition is marked; the join of that iteration is already running and still completes, later iterations skip it.
    bool converged = false;
    // As shipped, update_segment_graph receives the partition's length where it expects the end of its row range
    // (:1276-1279 against :1129-1135): rows [start, length) of the whole build are updated, i.e. the first
    // length - start rows of the partition, none at all once start >= length.
    const uint32_t shipped_rows = shipped ? (n > row_index_base ? n - row_index_base : 0u) : 0xffffffffu;
    for (uint32_t it = 0; it < iterations && !converged; it++) {
        if (shipped) shipped->last_join = it;
        cur_old = P.fwd_old;            // upload of h_graph_old / list sizes (:1290-1302)
        n_cur_old = P.n_fwd_old;
        if (it > 0) {                   // update_and_sample (:1270-1284)
            const int64_t counter = update_lists(P, host_ids, host_dists, row_index_base, shipped_rows, shipped != nullptr);
            if (static_cast<float>(counter) < termination_limit) converged = true;
        }
        sample_lists(P, false);
        std::vector<int> next_old = P.fwd_old;
        std::vector<uint32_t> n_next_old = P.n_fwd_old;
        P.fwd_old = cur_old;
        P.n_fwd_old = n_cur_old;
        reverse_lists(n, P.fwd_new, P.n_fwd_new, P.rev_new, P.n_rev_new);
        reverse_lists(n, P.fwd_old, P.n_fwd_old, P.rev_old, P.n_rev_old);
        std::fill(P.dev_dists.begin(), P.dev_dists.end(), FLT_MAX);   // local_join nn_descent.cuh:1217-1220
#pragma omp parallel
        {
            std::vector<float> xn(static_cast<size_t>(kBi) * dim), xo(static_cast<size_t>(kBi) * dim), D(kBi * kBi);
#pragma omp for schedule(dynamic, 64)
            for (int64_t L = 0; L < static_cast<int64_t>(n); L++) local_join(P, static_cast<uint32_t>(L), xn, xo, D);
        }
        P.fwd_old = next_old;
        P.n_fwd_old = n_next_old;
        // As shipped, the loop is left before the download once every partition is marked (:1344-1351): the results of the
        // joins of that iteration are never seen by the host.
        if (shipped && it >= shipped->break_iteration) break;
        host_ids = P.dev_ids;           // download (:1353-1361)
        host_dists = P.dev_dists;
        // new samples = downloaded entries not yet seen by the Bloom filter (sample_graph_new :973-1001)
#pragma omp parallel for schedule(static)
        for (int64_t i = 0; i < static_cast<int64_t>(n); i++) {
            uint32_t c = 0;
            for (uint32_t j = 0; j < kSeg; j++) {
                int &e = host_ids[static_cast<size_t>(i) * kSeg + j];
                uint32_t nid = static_cast<uint32_t>(id_of(e));
                if (nid >= n) break;
                if (bloom.check_add(static_cast<uint32_t>(i), nid)) continue;
                e = mark_old(e);
                P.fwd_new[static_cast<size_t>(i) * kSamples + c++] = static_cast<int>(nid);
                if (c == kSamples) break;
            }
            P.n_fwd_new[i] = c;
        }
    }
    update_lists(P, host_ids, host_dists, row_index_base, 0xffffffffu, shipped != nullptr);  // nn_descent.cuh:1368: every row, the last download
    if (shipped) {
        // shrink as shipped (:1376-1402): the first K columns of the row as stored, sub-list after sub-list, no sort across
        // sub-lists -- for K > 32 no id of the last sub-list (id % num_sub == num_sub - 1) is ever returned
#pragma omp parallel for schedule(static)
        for (int64_t i = 0; i < static_cast<int64_t>(n); i++) {
            for (uint32_t j = 0; j < K; j++) {
                const uint32_t idx = (row_index_base + static_cast<uint32_t>(i)) * P.W + j;
                const uint32_t id = static_cast<uint32_t>(id_of(P.lists[static_cast<size_t>(i) * P.W + j]));
                out[static_cast<size_t>(i) * K + j] = id < n ? static_cast<int>(id) : static_cast<int>(go_xorshift32(idx) % n);
            }
        }
        for (auto &l : P.locks) omp_destroy_lock(&l);
        return;
    }

    // shrink nn_descent.cuh:1376-1402.  For K > 32 the reference copies whole sub-lists in storage order and
    // therefore never returns ids with id % num_sub == num_sub-1; here sub-lists are merged by distance first.
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < static_cast<int64_t>(n); i++) {
        std::vector<std::pair<float, int>> row;
        for (uint32_t j = 0; j < P.W; j++) {
            int v = P.lists[static_cast<size_t>(i) * P.W + j];
            uint32_t id = static_cast<uint32_t>(id_of(v));
            if (id < n) row.emplace_back(P.ldists[static_cast<size_t>(i) * P.W + j], static_cast<int>(id));
        }
        if (P.num_sub > 1) std::stable_sort(row.begin(), row.end());
        for (uint32_t j = 0; j < K; j++) {
            uint32_t idx = (row_index_base + static_cast<uint32_t>(i)) * P.W + j;
            out[static_cast<size_t>(i) * K + j] = j < row.size() ? row[j].second : static_cast<int>(go_xorshift32(idx) % n);
        }
    }
    for (auto &l : P.locks) omp_destroy_lock(&l);
}

}  // namespace

extern "C" int go_nnd_build_ex(const float *reorder_data, uint32_t reorder_num, uint32_t dim,
                               const uint32_t *segment_starts, const uint32_t *segment_lengths, uint32_t segment_num,
                               uint32_t knn_degree, uint32_t iterations, float termination_threshold, uint32_t seed,
                               int32_t *knn_graph, int threads) {
#ifdef _OPENMP
    if (threads > 0) omp_set_num_threads(threads);
#endif
    if (knn_degree == 0 || knn_degree > 256) return -1;
    // preprocess_data_kernel nn_descent.cuh:445-488: rows stored as halfs, squared norms taken from the fp32 input
    std::vector<float> half(static_cast<size_t>(reorder_num) * dim), norms(reorder_num);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < static_cast<int64_t>(reorder_num); i++) {
        float acc = 0.0f;
        for (uint32_t t = 0; t < dim; t++) {
            float v = reorder_data[static_cast<size_t>(i) * dim + t];
            acc += v * v;
            half[static_cast<size_t>(i) * dim + t] = round_half(v);
        }
        norms[i] = acc;
    }
    for (uint32_t s = 0; s < segment_num; s++) {
        uint32_t start = segment_starts[s], len = segment_lengths[s];
        if (len == 0) continue;
        if (start + len > reorder_num) return -2;
        // termination_threshold * nrow * dim / counter_interval with nrow = all rows of the build (nn_descent.cuh:1280)
        const float limit = termination_threshold * static_cast<float>(reorder_num) * static_cast<float>(dim) / 100.0f;
        build_partition(half.data() + static_cast<size_t>(start) * dim, norms.data() + start, len, dim, knn_degree, iterations, seed,
                        knn_graph + static_cast<size_t>(start) * knn_degree, start, limit);
    }
    return 0;
}

// go_nnd_build_ex from given start lists: reorder_num x extended degree partition-local ids, a row's sub-lists one after
// the other (sub-list s holds ids with id % num_sub == s), negative = empty slot.
extern "C" int go_nnd_build_from(const float *reorder_data, uint32_t reorder_num, uint32_t dim, const uint32_t *segment_starts,
                                 const uint32_t *segment_lengths, uint32_t segment_num, uint32_t knn_degree, uint32_t iterations,
                                 float termination_threshold, const int32_t *start_lists, int32_t *knn_graph, int threads) {
#ifdef _OPENMP
    if (threads > 0) omp_set_num_threads(threads);
#endif
    if (knn_degree == 0 || knn_degree > 256 || !start_lists) return -1;
    const uint32_t W = go_nnd_extended_degree(knn_degree);
    std::vector<float> half(static_cast<size_t>(reorder_num) * dim), norms(reorder_num);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < static_cast<int64_t>(reorder_num); i++) {
        float acc = 0.0f;
        for (uint32_t t = 0; t < dim; t++) {
            float v = reorder_data[static_cast<size_t>(i) * dim + t];
            acc += v * v;
            half[static_cast<size_t>(i) * dim + t] = round_half(v);
        }
        norms[i] = acc;
    }
    for (uint32_t s = 0; s < segment_num; s++) {
        uint32_t start = segment_starts[s], len = segment_lengths[s];
        if (len == 0) continue;
        if (start + len > reorder_num) return -2;
        const float limit = termination_threshold * static_cast<float>(reorder_num) * static_cast<float>(dim) / 100.0f;
        build_partition(half.data() + static_cast<size_t>(start) * dim, norms.data() + start, len, dim, knn_degree, iterations, 0,
                        knn_graph + static_cast<size_t>(start) * knn_degree, start, limit, nullptr, start_lists + static_cast<size_t>(start) * W);
    }
    return 0;
}

extern "C" int go_nnd_build(const float *reorder_data, uint32_t reorder_num, uint32_t dim,
                            const uint32_t *segment_starts, const uint32_t *segment_lengths, uint32_t segment_num,
                            uint32_t knn_degree, uint32_t iterations, uint32_t seed, int32_t *knn_graph,
                            int threads) {
    return go_nnd_build_ex(reorder_data, reorder_num, dim, segment_starts, segment_lengths, segment_num, knn_degree, iterations, 0.0f,
                           seed, knn_graph, threads);
}

// The NN-descent build as the reference ships it: partitions whose first row index is not below their length are never
// updated between rounds, count no insertions, are marked converged after the first update step and get two rounds of
// joins; the partition-local id is compared with the row's index in the whole build; the sub-lists are not merged before
// truncation.  termination_threshold as in NNDescentParameter (1e-4).  Two passes: the first finds the iteration at which
// each partition is marked, the second knows when the loop was left.
extern "C" int go_nnd_build_shipped(const float *reorder_data, uint32_t reorder_num, uint32_t dim, const uint32_t *segment_starts,
                                    const uint32_t *segment_lengths, uint32_t segment_num, uint32_t knn_degree, uint32_t iterations,
                                    float termination_threshold, uint32_t seed, int32_t *knn_graph, int threads) {
#ifdef _OPENMP
    if (threads > 0) omp_set_num_threads(threads);
#endif
    if (knn_degree == 0 || knn_degree > 256) return -1;
    std::vector<float> half(static_cast<size_t>(reorder_num) * dim), norms(reorder_num);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < static_cast<int64_t>(reorder_num); i++) {
        float acc = 0.0f;
        for (uint32_t t = 0; t < dim; t++) {
            float v = reorder_data[static_cast<size_t>(i) * dim + t];
            acc += v * v;
            half[static_cast<size_t>(i) * dim + t] = round_half(v);
        }
        norms[i] = acc;
    }
    const float limit = termination_threshold * static_cast<float>(reorder_num) * static_cast<float>(dim) / 100.0f;
    uint32_t break_iteration = 0;
    for (int pass = 0; pass < 2; pass++) {
        for (uint32_t s = 0; s < segment_num; s++) {
            uint32_t start = segment_starts[s], len = segment_lengths[s];
            if (len == 0) continue;
            if (start + len > reorder_num) return -2;
            Shipped sh{pass == 0 ? iterations : break_iteration, 0};
            build_partition(half.data() + static_cast<size_t>(start) * dim, norms.data() + start, len, dim, knn_degree, iterations, seed,
                            knn_graph + static_cast<size_t>(start) * knn_degree, start, limit, &sh);
            if (pass == 0) break_iteration = std::max(break_iteration, sh.last_join);
        }
        // the loop runs all its iterations unless every partition was marked before the last one
        if (pass == 0 && break_iteration + 1 >= iterations) break_iteration = iterations;
    }
    return 0;
}
