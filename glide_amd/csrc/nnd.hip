// NN-descent kNN-graph construction, entirely on the device.
//
// Reference: nn_descent.cuh -- preprocess_data_kernel (:445-488), sampling on the host (GnndGraph::sample_graph
// :1040-1071, sample_graph_new :973-1001), add_rev_edges_kernel (:490-507), local_join_kernel (:668-914),
// insert_to_global_graph (:509-579), host merge update_graph (:1106-1126) and the shrink step (:1376-1402).
//
// What is kept: fp16 rows with fp32 squared norms, <= 32 new + <= 32 old forward samples per node, reverse
// samples capped at 32, a 64 x 64 distance tile per phase (new x new, new x old) computed on the matrix cores
// with the norm-trick epilogue, and one offer per row / column (its nearest partner) per phase.
// What is different: the kNN lists, flags and samples never leave HBM.  Offers are appended to a per-node inbox
// (one atomic counter per node, no locks, no cross-workgroup read-after-write inside a kernel) and a merge kernel
// folds each inbox into the node's sorted list with a wave-wide bitonic sort; sampling uses the new/old flag kept
// in the list instead of a host-side Bloom filter.  All ids are partition-local.
#include "common.hpp"
#include "host_util.hpp"
#include <vector>

namespace glide {

typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));

constexpr uint32_t kSamples = 32;     // NUM_SAMPLES (nn_descent.cuh:391)
constexpr uint32_t kBi = 64;          // MAX_NUM_BI_SAMPLES (:392)
constexpr uint32_t kOld = 0x80000000u;  // "old" flag in a list entry (the reference uses the sign bit, :53-72)
constexpr int kJoinChunk = 64;         // dims staged per step of the join
constexpr int kRowHalfs = kJoinChunk + 8;   // LDS row stride in halfs for one chunk
constexpr int kDStride = 65;

struct Segments {
    const uint32_t* starts;
    const uint32_t* lengths;
    uint32_t count;
    uint32_t* state;     // per partition: kActive, kLastRound (one more join, as the reference's overlapped loop does), kDone
    uint32_t* updates;   // per partition: list insertions seen on every 100th row in the current round
};
constexpr uint32_t kActive = 0, kLastRound = 1, kDone = 2;
constexpr uint32_t kMaxSegments = 2048;
constexpr uint32_t kCounterInterval = 100;   // counter_interval, nn_descent.cuh:1123

__device__ __forceinline__ void locate(const Segments& s, uint32_t node, uint32_t& start, uint32_t& len) {
    uint32_t i = 0;
    for (; i + 1 < s.count; i++)
        if (node < s.starts[i] + s.lengths[i]) break;
    start = s.starts[i];
    len = s.lengths[i];
}

// Same result for a node every lane of the wavefront shares: the lanes test one segment each, so the lookup costs
// one memory round trip instead of one per segment.  Every lane of the wavefront must call it.  Returns the index.
__device__ __forceinline__ uint32_t locate_uniform(const Segments& s, uint32_t node, uint32_t& start, uint32_t& len) {
    uint32_t found = s.count - 1;
    for (uint32_t base = 0; base + 1 < s.count; base += 64) {
        const uint32_t i = base + lane_id();
        const bool hit = i + 1 < s.count && node < s.starts[i] + s.lengths[i];
        const uint64_t m = ballot(hit);
        if (m) {
            found = base + static_cast<uint32_t>(__ffsll(static_cast<long long>(m))) - 1;
            break;
        }
    }
    start = s.starts[found];
    len = s.lengths[found];
    return found;
}

// ---- prepare: fp32 rows -> fp16 rows (stride dim_pad, zero padded) + squared norms of the fp32 input
__global__ __launch_bounds__(256) void nnd_prepare_kernel(const float* data, uint32_t num, uint32_t dim, uint32_t dim_pad, _Float16* half_rows,
                                                          float* norms) {
    const int lane = lane_id();
    const uint32_t i = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (i >= num) return;
    float acc = 0.f;
    for (uint32_t d = lane; d < dim_pad; d += 64) {
        const float v = d < dim ? data[static_cast<size_t>(i) * dim + d] : 0.f;
        acc = fmaf(v, v, acc);
        half_rows[static_cast<size_t>(i) * dim_pad + d] = static_cast<_Float16>(v);
    }
    acc = wave_sum(acc);
    if (lane == 0) norms[i] = acc;
}

// ---- random initial lists.  The reference (init_random_graph :1003-1038) shuffles one sequence of len / num_sub values
// per sub-list on the host and hands out consecutive runs of it: entry j of sub-list `sub` of node i is
// seq_sub[(i * width + 32 * sub + j) % m] * num_sub + sub.  Every id therefore starts with the same in-degree and
// neighbouring nodes start with disjoint lists, which shapes the first rounds; the same construction is used here,
// with a keyed bijection (a cycle-walking Feistel network) in place of the host-side shuffle.
__device__ __forceinline__ uint32_t mix32(uint32_t x) {
    x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
    return x;
}

// A permutation of [0, m): four Feistel rounds on the smallest even number of bits covering m, re-applied until the
// value falls below m (at most 4 m values in the domain, so a few rounds on average; every walk ends because the
// network is a bijection of the domain).
__device__ __forceinline__ uint32_t permute(uint32_t x, uint32_t m, uint32_t key) {
    if (m <= 1) return 0;
    uint32_t bits = 32 - __clz(m - 1);
    bits = bits < 2 ? 2 : (bits + 1) & ~1u;
    const uint32_t half = bits / 2, mask = (1u << half) - 1;
    do {
        uint32_t l = x >> half, r = x & mask;
#pragma unroll
        for (uint32_t round = 0; round < 4; round++) {
            const uint32_t t = l ^ (mix32(r ^ (key + round * 0x9E3779B9u)) & mask);
            l = r;
            r = t;
        }
        x = (l << half) | r;
    } while (x >= m);
    return x;
}

__global__ __launch_bounds__(256) void nnd_init_kernel(uint32_t* list_ids, float* list_dists, uint32_t* inbox_counts, uint32_t num, uint32_t width,
                                                       Segments segs, uint32_t seed) {
    const uint32_t idx = blockIdx.x * 256 + threadIdx.x;
    const uint32_t node = idx / width, j = idx % width;
    if (node >= num) return;
    uint32_t start, len;
    locate(segs, node, start, len);
    const uint32_t local = node - start;
    const uint32_t num_sub = width / kSamples, sub = j / kSamples;
    const uint32_t m = len / num_sub > 1 ? len / num_sub : 1;
    const uint32_t key = mix32(seed * 7919u + sub + 0x5bd1e995u * start);
    const uint32_t at = local * width + j;
    uint32_t id = permute(at % m, m, key) * num_sub + sub;
    if (id == local) id = permute((at + kSamples) % m, m, key) * num_sub + sub;
    if (id >= len || id == local) id = kInvalid;   // partitions too small to fill a list
    // stored column-major over the sub-lists, the order in which the first samples are taken (:1052-1068)
    const uint32_t slot = (j % kSamples) * num_sub + sub;
    list_ids[static_cast<size_t>(node) * width + slot] = id;   // new (flag clear)
    list_dists[static_cast<size_t>(node) * width + slot] = FLT_MAX;
    if (j == 0) inbox_counts[node] = 0;
}

// ---- sampling: first <= 32 new entries (marked old afterwards) and first <= 32 entries that were already old
__global__ __launch_bounds__(256) void nnd_sample_kernel(uint32_t* list_ids, uint32_t num, uint32_t width, Segments segs, uint32_t* fwd_new,
                                                         uint32_t* fwd_old, uint32_t* counts /* num x 4: fwd_new, fwd_old, rev_new, rev_old */) {
    const int lane = lane_id();
    const uint32_t node = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (node >= num) return;
    uint32_t start, len;
    locate_uniform(segs, node, start, len);
    uint32_t nn = 0, no = 0;
    for (uint32_t base = 0; base < width; base += 64) {
        const uint32_t j = base + lane;
        uint32_t e = j < width ? list_ids[static_cast<size_t>(node) * width + j] : kInvalid;
        const uint32_t id = e & ~kOld;
        const bool valid = e != kInvalid && id < len;
        const bool is_new = valid && (e & kOld) == 0;
        const bool is_old = valid && (e & kOld) != 0;
        const uint64_t mn = ballot(is_new), mo = ballot(is_old);
        const uint32_t pn = nn + prefix_count(mn), po = no + prefix_count(mo);
        if (is_new && pn < kSamples) {
            fwd_new[static_cast<size_t>(node) * kSamples + pn] = id;
            list_ids[static_cast<size_t>(node) * width + j] = e | kOld;
        }
        if (is_old && po < kSamples) fwd_old[static_cast<size_t>(node) * kSamples + po] = id;
        nn += __popcll(mn);
        no += __popcll(mo);
    }
    if (lane == 0) {
        counts[static_cast<size_t>(node) * 4 + 0] = nn < kSamples ? nn : kSamples;
        counts[static_cast<size_t>(node) * 4 + 1] = no < kSamples ? no : kSamples;
        counts[static_cast<size_t>(node) * 4 + 2] = 0;
        counts[static_cast<size_t>(node) * 4 + 3] = 0;
    }
}

// ---- reverse samples (add_rev_edges_kernel :490-507): list u appends itself to the reverse list of each sample
__global__ __launch_bounds__(256) void nnd_reverse_kernel(const uint32_t* fwd_new, const uint32_t* fwd_old, uint32_t* counts, uint32_t* rev_new,
                                                          uint32_t* rev_old, uint32_t num, Segments segs) {
    const uint32_t idx = blockIdx.x * 256 + threadIdx.x;
    const uint32_t node = idx / 64, j = idx % 64;
    if (node >= num) return;
    uint32_t start, len;
    const uint32_t seg = locate_uniform(segs, node, start, len);
    if (segs.state[seg] == kDone) return;
    const uint32_t which = j / kSamples, k = j % kSamples;   // 0: new, 1: old
    if (k >= counts[static_cast<size_t>(node) * 4 + which]) return;
    const uint32_t v = (which ? fwd_old : fwd_new)[static_cast<size_t>(node) * kSamples + k];
    const uint32_t target = start + v;
    const uint32_t pos = atomicAdd(&counts[static_cast<size_t>(target) * 4 + 2 + which], 1u);
    if (pos < kSamples) (which ? rev_old : rev_new)[static_cast<size_t>(target) * kSamples + pos] = node - start;
}

// ---- local join ---------------------------------------------------------------------------------------------
struct JoinArgs {
    const _Float16* half_rows;
    const float* norms;
    const uint32_t* fwd_new;
    const uint32_t* fwd_old;
    const uint32_t* rev_new;
    const uint32_t* rev_old;
    uint32_t* counts;           // num x 4: forward new / old, reverse new / old
    uint32_t* inbox_counts;
    uint2* inbox;               // num x inbox_cap (dist bits, id)
    unsigned long long* stats;  // [0] offers emitted, [1] offers dropped by a full inbox (nullable)
    uint32_t num, dim_pad, width, inbox_cap;
    Segments segs;
};

struct JoinRows {
    _Float16 xn[kBi][kRowHalfs];
    _Float16 xo[kBi][kRowHalfs];
};
struct JoinLds {
    union {               // the distance tile is written only after the last matrix-core pass has read the rows
        JoinRows rows;
        float dist[kBi][kDStride];
    };
    uint32_t new_ids[kBi], old_ids[kBi];
    float new_norms[kBi], old_norms[kBi];
    uint32_t hash_new[128], hash_old[128];
    uint32_t n_new, n_old;
};

__device__ __forceinline__ bool lds_set_insert(uint32_t* table, uint32_t key) {   // 128-slot open addressing
    uint32_t idx = (key * 0x9E3779B1u) >> 25;
    for (int i = 0; i < 128; i++) {
        const uint32_t old = atomicCAS(&table[idx], kInvalid, key);
        if (old == kInvalid) return true;
        if (old == key) return false;
        idx = (idx + 1) & 127;
    }
    return false;
}

// No filtering of offers against the target's current list: the reference also explores offers that do not enter
// the list (they are the "new" samples of the next round, nn_descent.cuh:973-1001).

// A (rows) x B (rows) dot products of one chunk of dims for this wave's 32 x 32 quadrant.
// v_mfma_f32_32x32x16_f16 (gfx950): lane supplies A[i = lane%32][k = 8*(lane/32) .. +7] and B[k = same][j = lane%32].
__device__ __forceinline__ void mfma_chunk(float16v& acc, const _Float16 (*A)[kRowHalfs], const _Float16 (*B)[kRowHalfs], int rb, int cb, int lane) {
    const int t = lane & 31, kh = lane >> 5;
#pragma unroll
    for (int kk = 0; kk < kJoinChunk; kk += 16) {
        const half8v av = *reinterpret_cast<const half8v*>(&A[rb * 32 + t][kk + 8 * kh]);
        const half8v bv = *reinterpret_cast<const half8v*>(&B[cb * 32 + t][kk + 8 * kh]);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, bv, acc, 0, 0, 0);
    }
}

// Nearest partner of one row (BY_ROW) or one column of the distance tile (get_min_item, nn_descent.cuh:581-623):
// four adjacent lanes scan 16 entries each, then combine (smaller distance, then smaller index).  Thread t handles
// line t/4.  Entries that must not win (outside the lists, the line's own id) hold FLT_MAX in the tile.
template <bool BY_ROW>
__device__ __forceinline__ void line_argmin(const float (*dist)[kDStride], uint32_t line, uint32_t part, float& best, uint32_t& best_idx) {
    best = FLT_MAX;
    best_idx = kInvalid;
    const uint32_t first = part * 16;
#pragma unroll
    for (uint32_t k = 0; k < 16; k++) {
        const uint32_t idx = first + k;
        const float d = BY_ROW ? dist[line][idx] : dist[idx][line];
        if (d < best) {
            best = d;
            best_idx = idx;
        }
    }
#pragma unroll
    for (int m = 1; m <= 2; m <<= 1) {
        const float od = m == 1 ? lane_xor<1>(best) : lane_xor<2>(best);
        const uint32_t oi = m == 1 ? lane_xor<1>(best_idx) : lane_xor<2>(best_idx);
        if (od < best || (od == best && oi < best_idx)) {
            best = od;
            best_idx = oi;
        }
    }
}

// Six workgroups per CU (80 registers per lane, 20 KB of LDS each): the join is bound by the latency of its
// gather -> matrix -> arg-min -> offer chain, so residency matters more than registers; seven would spill.
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(6, 6))) void nnd_join_kernel(JoinArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    JoinLds& L = *reinterpret_cast<JoinLds*>(smem);
    const uint32_t node = blockIdx.x;
    if (node >= a.num) return;
    const int tid = threadIdx.x, lane = lane_id(), wave = tid >> 6;

    // sample ids are fetched before the counts are known (one memory round trip instead of two)
    uint32_t my_id = kInvalid;
    if (tid < 128) {
        const bool is_old = tid >= 64;
        const uint32_t k = tid & 63;
        const uint32_t* src = k < kSamples ? (is_old ? a.fwd_old : a.fwd_new) : (is_old ? a.rev_old : a.rev_new);
        my_id = src[static_cast<size_t>(node) * kSamples + (k & (kSamples - 1))];
        L.hash_new[tid] = kInvalid;
        L.hash_old[tid] = kInvalid;
    }
    const uint4 c4 = *reinterpret_cast<const uint4*>(a.counts + static_cast<size_t>(node) * 4);
    uint32_t seg_start, seg_len;
    const uint32_t seg = locate_uniform(a.segs, node, seg_start, seg_len);
    if (a.segs.state[seg] == kDone) return;
    const uint32_t c_fn = c4.x, c_fo = c4.y;
    const uint32_t c_rn = c4.z < kSamples ? c4.z : kSamples, c_ro = c4.w < kSamples ? c4.w : kSamples;
    // The counts must have arrived in every thread before thread 0 restarts them below; the barrier itself waits
    // for LDS traffic only, so the registers are consumed here.
    asm volatile("" ::"v"(c4.x), "v"(c4.y), "v"(c4.z), "v"(c4.w));
    __syncthreads();
    // this list's reverse samples are consumed here and now: the counts restart for the scatter that follows the join
    if (tid == 0) *reinterpret_cast<uint2*>(a.counts + static_cast<size_t>(node) * 4 + 2) = make_uint2(0u, 0u);
    if (c_fn + c_rn == 0) return;
    // forward then reverse samples, duplicates removed with an LDS hash set (reference: sort + binary search, :625-666)
    if (tid < 128) {
        const bool is_old = tid >= 64;
        const uint32_t k = tid & 63;
        const uint32_t cf = is_old ? c_fo : c_fn, cr = is_old ? c_ro : c_rn;
        const bool present = k < kSamples ? k < cf : (k - kSamples) < cr;
        const uint32_t id = present ? my_id : kInvalid;
        const bool keep = id != kInvalid && id < seg_len && lds_set_insert(is_old ? L.hash_old : L.hash_new, id);
        const uint64_t m = ballot(keep);   // wave 0 = new, wave 1 = old; forward entries keep the lower ranks
        if (keep) {
            const uint32_t pos = prefix_count(m);
            (is_old ? L.old_ids : L.new_ids)[pos] = id;
        }
        if (lane == 0) (is_old ? L.n_old : L.n_new) = __popcll(m);
    }
    __syncthreads();
    const uint32_t n_new = L.n_new, n_old = L.n_old;
    if (n_new == 0) return;

    const int rb = wave >> 1, cb = wave & 1;
    float16v acc_nn, acc_no;
#pragma unroll
    for (int r = 0; r < 16; r++) {
        acc_nn[r] = 0.f;
        acc_no[r] = 0.f;
    }
    const bool need_nn = (rb * 32 < static_cast<int>(n_new)) && (cb * 32 < static_cast<int>(n_new));
    const bool need_no = (rb * 32 < static_cast<int>(n_new)) && (cb * 32 < static_cast<int>(n_old));

    // Chunks of kJoinChunk dims go global -> registers -> LDS: 8 lanes x 16 B per row and chunk, 32 rows per pass (new
    // rows, then old rows).  The loads of chunk k+1 are issued before the matrix instructions of chunk k.  Short chunks
    // keep the workgroup at 20 KB of LDS, so seven of them share a CU instead of four.
    float4 pre[4];
    auto prefetch = [&](uint32_t k0) {
#pragma unroll
        for (int pass = 0; pass < 4; pass++) {
            const uint32_t r = pass * 32 + (tid >> 3), q = tid & 7;
            const bool is_old = r >= 64;
            const uint32_t rr = r & 63;
            const uint32_t d0 = k0 + q * 8;
            pre[pass] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (rr < (is_old ? n_old : n_new)) {
                const uint32_t id = (is_old ? L.old_ids : L.new_ids)[rr];
                if (d0 < a.dim_pad) pre[pass] = *reinterpret_cast<const float4*>(a.half_rows + static_cast<size_t>(seg_start + id) * a.dim_pad + d0);
                if (k0 == 0 && q == 0) (is_old ? L.old_norms : L.new_norms)[rr] = a.norms[seg_start + id];   // same round trip as the row
            }
        }
    };
    prefetch(0);
    for (uint32_t k0 = 0; k0 < a.dim_pad; k0 += kJoinChunk) {
        if (k0) __syncthreads();   // every wave is done with the previous chunk
#pragma unroll
        for (int pass = 0; pass < 4; pass++) {
            const uint32_t r = pass * 32 + (tid >> 3), q = tid & 7;
            *reinterpret_cast<float4*>(&(r >= 64 ? L.rows.xo : L.rows.xn)[r & 63][q * 8]) = pre[pass];
        }
        __syncthreads();
        if (k0 + kJoinChunk < a.dim_pad) prefetch(k0 + kJoinChunk);
        if (need_nn) mfma_chunk(acc_nn, L.rows.xn, L.rows.xn, rb, cb, lane);
        if (need_no) mfma_chunk(acc_no, L.rows.xn, L.rows.xo, rb, cb, lane);
    }

    const int t = lane & 31, kh = lane >> 5;
    const uint32_t line = tid >> 2, part = tid & 3;
    // ---- phase 1: new x new
    __syncthreads();   // every wave is done with the rows: the tile may overwrite them
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const uint32_t i = rb * 32 + 8 * (r / 4) + 4 * kh + (r % 4), j = cb * 32 + t;
        float d = FLT_MAX;
        if (i < n_new && j < n_new && i != j) d = fmaxf((L.new_norms[i] + L.new_norms[j]) - 2.f * acc_nn[r], 0.f);
        L.dist[i][j] = d;
    }
    __syncthreads();
    // offers are collected first and sent at the end, so their atomics overlap instead of costing a round trip each
    uint32_t off_target[3] = {kInvalid, kInvalid, kInvalid}, off_cand[3] = {kInvalid, kInvalid, kInvalid};
    float off_dist[3] = {FLT_MAX, FLT_MAX, FLT_MAX};
    {
        float best;
        uint32_t bj;
        line_argmin<true>(L.dist, line, part, best, bj);
        if (part == 0 && line < n_new && bj != kInvalid) {
            off_target[0] = L.new_ids[line];
            off_cand[0] = L.new_ids[bj];
            off_dist[0] = best;
        }
    }
    if (n_old != 0) {
        // ---- phase 2: new x old (rows: new, columns: old)
        __syncthreads();
        const uint32_t col_id = cb * 32 + t < n_old ? L.old_ids[cb * 32 + t] : kInvalid;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const uint32_t i = rb * 32 + 8 * (r / 4) + 4 * kh + (r % 4), j = cb * 32 + t;
            float d = FLT_MAX;   // also where the same point sits in both lists: it is no partner of itself
            if (i < n_new && j < n_old && L.new_ids[i] != col_id) d = fmaxf((L.new_norms[i] + L.old_norms[j]) - 2.f * acc_no[r], 0.f);
            L.dist[i][j] = d;
        }
        __syncthreads();
        {
            float best;
            uint32_t bj;
            const uint32_t me = line < n_new ? L.new_ids[line] : kInvalid;
            line_argmin<true>(L.dist, line, part, best, bj);
            if (part == 0 && line < n_new && bj != kInvalid) {
                off_target[1] = me;
                off_cand[1] = L.old_ids[bj];
                off_dist[1] = best;
            }
        }
        {
            float best;
            uint32_t bi;
            const uint32_t me = line < n_old ? L.old_ids[line] : kInvalid;
            line_argmin<false>(L.dist, line, part, best, bi);
            if (part == 0 && line < n_old && bi != kInvalid) {
                off_target[2] = me;
                off_cand[2] = L.new_ids[bi];
                off_dist[2] = best;
            }
        }
    }
    uint32_t pos[3];
#pragma unroll
    for (int k = 0; k < 3; k++) {
        const bool ok = off_cand[k] != kInvalid && off_cand[k] != off_target[k] && off_cand[k] < seg_len && off_dist[k] < FLT_MAX;
        if (!ok) off_target[k] = kInvalid;
        pos[k] = ok ? atomicAdd(&a.inbox_counts[seg_start + off_target[k]], 1u) : kInvalid;
    }
#pragma unroll
    for (int k = 0; k < 3; k++) {
        if (off_target[k] != kInvalid && pos[k] < a.inbox_cap)
            a.inbox[static_cast<size_t>(seg_start + off_target[k]) * a.inbox_cap + pos[k]] = make_uint2(__float_as_uint(off_dist[k]), off_cand[k]);
    }
}

// ---- merge: list (width) + inbox (<= cap) -> sorted, de-duplicated list of `width`; one wavefront per node
// key = dist bits : id (31 bits) : source (0 = already in the list, 1 = offer); payload = old flag
template <int M>
struct Net64 {
    static constexpr int NR = M / 64;
    template <int LM>
    static __device__ __forceinline__ unsigned long long xor_lane(unsigned long long v) {
        const uint32_t lo = lane_xor<LM>(static_cast<uint32_t>(v)), hi = lane_xor<LM>(static_cast<uint32_t>(v >> 32));
        return (static_cast<unsigned long long>(hi) << 32) | lo;
    }
    template <int K, int J>
    static __device__ __forceinline__ void stage(unsigned long long (&k)[NR], uint32_t (&v)[NR], int lane) {
        if constexpr (J < NR) {
#pragma unroll
            for (int r = 0; r < NR; r++) {
                if ((r & J) == 0) {
                    const int e = NR * lane + r;
                    const bool asc = (K >= M) ? true : ((e & K) == 0);
                    if ((k[r] > k[r | J]) == asc) {
                        const unsigned long long tk = k[r]; k[r] = k[r | J]; k[r | J] = tk;
                        const uint32_t tv = v[r]; v[r] = v[r | J]; v[r | J] = tv;
                    }
                }
            }
        } else {
            // Two entries with equal keys are copies of one offer (same distance, id, source and flag), so exchanging
            // them or not gives the same sequence: one compare decides, and the lanes that keep the larger key take the
            // partner's entry exactly where the others would not (the complement of the compare mask).
            constexpr int LM = J / NR;
#pragma unroll
            for (int r = 0; r < NR; r++) {
                uint64_t keep_min = 0;   // compile-time pattern: lower partner of an ascending pair, upper of a descending one
                for (int l = 0; l < 64; l++) {
                    const int e = NR * l + r;
                    const bool asc = (K >= M) ? true : ((e & K) == 0);
                    if (((l & LM) == 0) == asc) keep_min |= 1ull << l;
                }
                const unsigned long long ok = xor_lane<LM>(k[r]);
                const uint32_t ov = lane_xor<LM>(v[r]);
                const uint64_t less = __builtin_amdgcn_ballot_w64(ok < k[r]);
                const uint64_t take = less ^ ~keep_min;
                const uint32_t lo = select_by_mask(static_cast<uint32_t>(k[r]), static_cast<uint32_t>(ok), take);
                const uint32_t hi = select_by_mask(static_cast<uint32_t>(k[r] >> 32), static_cast<uint32_t>(ok >> 32), take);
                k[r] = (static_cast<unsigned long long>(hi) << 32) | lo;
                v[r] = select_by_mask(v[r], ov, take);
            }
        }
    }
    template <int K, int J>
    static __device__ __forceinline__ void merge_from(unsigned long long (&k)[NR], uint32_t (&v)[NR], int lane) {
        stage<K, J>(k, v, lane);
        if constexpr (J > 1) merge_from<K, J / 2>(k, v, lane);
    }
    template <int K>
    static __device__ __forceinline__ void sort_from(unsigned long long (&k)[NR], uint32_t (&v)[NR], int lane) {
        merge_from<K, K / 2>(k, v, lane);
        if constexpr (K < M) sort_from<K * 2>(k, v, lane);
    }
    static __device__ __forceinline__ void sort(unsigned long long (&k)[NR], uint32_t (&v)[NR], int lane) { sort_from<2>(k, v, lane); }
};

// Bloom filter of ids already used as "new" samples (reference BloomFilter :203-276: 512-bit sets, 3 hashes)
__device__ __forceinline__ uint32_t bloom_h0(uint32_t v) { v *= 1103515245u; v += 12345u; v ^= v << 13; v ^= v >> 17; v ^= v << 5; return v; }
__device__ __forceinline__ uint32_t bloom_h1(uint32_t v) { v *= 1664525u; v += 1013904223u; v ^= v << 13; v ^= v >> 17; v ^= v << 5; return v; }

// Prefix sum over the 64 lanes without LDS traffic: four shifted adds inside each row of 16 lanes, then lane 15 of a row
// is added to the next row (rows 1 and 3) and lane 31 to the upper half (rows 2 and 3).  Lanes a step does not feed add 0.
__device__ __forceinline__ uint32_t wave_exclusive_scan(uint32_t value, int lane, uint32_t& total) {
    (void) lane;
    int x = static_cast<int>(value);
    x += __builtin_amdgcn_update_dpp(0, x, 0x111, 0xf, 0xf, true);   // row_shr:1
    x += __builtin_amdgcn_update_dpp(0, x, 0x112, 0xf, 0xf, true);   // row_shr:2
    x += __builtin_amdgcn_update_dpp(0, x, 0x114, 0xf, 0xf, true);   // row_shr:4
    x += __builtin_amdgcn_update_dpp(0, x, 0x118, 0xf, 0xf, true);   // row_shr:8
    x += __builtin_amdgcn_update_dpp(0, x, 0x142, 0xa, 0xf, true);   // row_bcast:15
    x += __builtin_amdgcn_update_dpp(0, x, 0x143, 0xc, 0xf, true);   // row_bcast:31
    total = static_cast<uint32_t>(__builtin_amdgcn_readlane(x, 63));
    return static_cast<uint32_t>(x) - value;
}

// Merge + resample, one wavefront per node.  The reference keeps, per node and round, a 32-wide sorted "device" list of
// the offers (insert_to_global_graph :509-579), merges it into the host list (update_graph :1106-1126) and draws the
// samples of the next join from both (sample_graph_new :973-1001, sample_segment_graph :1073-1104).  Here:
//   old samples = the first <= 32 entries of the incoming list that are flagged old (the reference samples them before
//                 this round's results are merged);
//   the list and this round's offers are sorted together by (distance, id); of the distinct offered ids only the
//   best 32 count (the rest are dropped, as the 32-wide device list drops them); those not yet in the list enter it;
//   new samples = those of the best 32 that the Bloom filter has not seen; the ones entering the list are flagged old.
// add_rev_edges_kernel (:490-507) for one sample: list `node` appends itself to the reverse list of sample `id`
__device__ __forceinline__ void reverse_append(uint32_t* counts, uint32_t* rev, uint32_t seg_start, uint32_t id, uint32_t which, uint32_t node) {
    const uint32_t target = seg_start + id;
    const uint32_t pos = atomicAdd(&counts[static_cast<size_t>(target) * 4 + which], 1u);
    if (pos < kSamples) rev[static_cast<size_t>(target) * kSamples + pos] = node - seg_start;
}

// The sort network is sized by what the node holds this round (list + offers received): the keys are distinct up to
// identical copies, so every size gives the same sorted sequence, and most nodes need far less than the largest one.
template <int M>
__device__ __forceinline__ void merge_node(uint32_t* list_ids, float* list_dists, uint32_t* inbox_counts, const uint2* inbox, uint32_t width,
                                           uint32_t inbox_cap, uint32_t* bloom, uint32_t bloom_sets, uint32_t* fwd_new, uint32_t* fwd_old,
                                           uint32_t* counts, unsigned long long* stats, Segments segs, uint32_t node, uint32_t seg, uint32_t raw,
                                           uint32_t* filter, int lane, uint32_t seg_start, uint32_t* rev_new, uint32_t* rev_old) {
    constexpr int NR = M / 64;
    const uint32_t bloom_words = bloom_sets * 16;
    const uint32_t n_in = raw < inbox_cap ? raw : inbox_cap;
    unsigned long long k[NR];
    uint32_t v[NR];
    uint32_t old_count = 0;
#pragma unroll
    for (int r = 0; r < NR; r++) {
        const uint32_t e = NR * lane + r;
        k[r] = ~0ull;
        v[r] = 0;
        if (e < width) {
            const uint32_t id = list_ids[static_cast<size_t>(node) * width + e];
            const float d = list_dists[static_cast<size_t>(node) * width + e];
            if (id != kInvalid) {
                k[r] = (static_cast<unsigned long long>(__float_as_uint(d)) << 32) | (static_cast<unsigned long long>(id & ~kOld) << 1);
                v[r] = id & kOld;
                old_count += (id & kOld) != 0;
            }
        } else if (e - width < n_in) {
            const uint2 o = inbox[static_cast<size_t>(node) * inbox_cap + (e - width)];
            k[r] = (static_cast<unsigned long long>(o.x) << 32) | (static_cast<unsigned long long>(o.y) << 1) | 1ull;
            v[r] = 0;   // offers enter as new
        }
    }
    // old samples from the incoming list (element order = list order)
    uint32_t total_old;
    {
        uint32_t rank = wave_exclusive_scan(old_count, lane, total_old);
#pragma unroll
        for (int r = 0; r < NR; r++) {
            if (k[r] != ~0ull && !(k[r] & 1ull) && (v[r] & kOld)) {
                if (rank < kSamples) {
                    const uint32_t id = static_cast<uint32_t>((k[r] >> 1) & 0x7fffffffull);
                    fwd_old[static_cast<size_t>(node) * kSamples + rank] = id;
                    if (rev_old) reverse_append(counts, rev_old, seg_start, id, 3, node);
                }
                rank++;
            }
        }
    }
    Net64<M>::sort(k, v, lane);
    // Equal id => equal distance => adjacent after the sort, the list's own copy first.  An id's first offered copy
    // represents the offer; it is "known" when the list already holds the id.
    bool from_list[NR], first_offer[NR], known[NR];
    uint32_t offer_count = 0;
    // the previous lane's last key (wave_shr:1; lane 0 has no predecessor and is handled as the head below)
    const unsigned long long last_of_prev =
        (static_cast<unsigned long long>(static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(k[NR - 1] >> 32), 0x138, 0xf, 0xf, false))) << 32) |
        static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(k[NR - 1]), 0x138, 0xf, 0xf, false));
#pragma unroll
    for (int r = 0; r < NR; r++) {
        const unsigned long long prev = r == 0 ? last_of_prev : k[r - 1];
        const bool head = (r == 0 && lane == 0);
        const bool valid = k[r] != ~0ull;
        const bool same_id = !head && (prev >> 1) == (k[r] >> 1);
        from_list[r] = valid && !(k[r] & 1ull) && !same_id;   // a repeated id inside the list (random start) is dropped
        first_offer[r] = valid && (k[r] & 1ull) && (!same_id || !(prev & 1ull));
        known[r] = first_offer[r] && same_id;
        offer_count += first_offer[r];
    }
    uint32_t total_offer, total_keep, total_new;
    uint32_t orank = wave_exclusive_scan(offer_count, lane, total_offer);
    bool keep[NR], fresh[NR];
    uint32_t keep_count = 0, fresh_count = 0;
#pragma unroll
    for (int r = 0; r < NR; r++) {
        fresh[r] = false;
        keep[r] = from_list[r];
        if (first_offer[r]) {
            if (orank < kSamples) {
                keep[r] = !known[r];
                const uint32_t id = static_cast<uint32_t>((k[r] >> 1) & 0x7fffffffull);
                const uint32_t base = (id % bloom_sets) * 512;
                uint32_t h = bloom_h0(id);
                const uint32_t b0 = base + h % 512;
                h += bloom_h1(id);
                const uint32_t b1 = base + h % 512;
                h += bloom_h1(id);
                const uint32_t b2 = base + h % 512;
                const bool seen = ((filter[b0 >> 5] >> (b0 & 31)) & (filter[b1 >> 5] >> (b1 & 31)) & (filter[b2 >> 5] >> (b2 & 31)) & 1u) != 0;
                fresh[r] = !seen;
            }
            orank++;
        }
        keep_count += keep[r];
        fresh_count += fresh[r];
    }
    uint32_t pos = wave_exclusive_scan(keep_count, lane, total_keep);
    uint32_t nrank = wave_exclusive_scan(fresh_count, lane, total_new);
    __builtin_amdgcn_wave_barrier();
    uint32_t inserted = 0;
#pragma unroll
    for (int r = 0; r < NR; r++) {
        const uint32_t id = static_cast<uint32_t>((k[r] >> 1) & 0x7fffffffull);
        uint32_t flag = v[r];
        if (fresh[r]) {   // at most 32 of them: all become samples
            fwd_new[static_cast<size_t>(node) * kSamples + nrank] = id;
            if (rev_new) reverse_append(counts, rev_new, seg_start, id, 2, node);
            nrank++;
            flag = kOld;
            const uint32_t base = (id % bloom_sets) * 512;
            uint32_t h = bloom_h0(id);
            const uint32_t b0 = base + h % 512;
            h += bloom_h1(id);
            const uint32_t b1 = base + h % 512;
            h += bloom_h1(id);
            const uint32_t b2 = base + h % 512;
            atomicOr(&filter[b0 >> 5], 1u << (b0 & 31));
            atomicOr(&filter[b1 >> 5], 1u << (b1 & 31));
            atomicOr(&filter[b2 >> 5], 1u << (b2 & 31));
        }
        if (keep[r]) {
            if (pos < width) {
                list_ids[static_cast<size_t>(node) * width + pos] = id | flag;
                list_dists[static_cast<size_t>(node) * width + pos] = __uint_as_float(static_cast<uint32_t>(k[r] >> 32));
                inserted += first_offer[r];
            }
            pos++;
        }
    }
    // update_counter (update_graph :1106-1126): insertions on every 100th row, per partition
    if (node % kCounterInterval == 0) {
        uint32_t total_inserted;
        wave_exclusive_scan(inserted, lane, total_inserted);
        if (lane == 0 && total_inserted) atomicAdd(&segs.updates[seg], total_inserted);
    }
    for (uint32_t e = total_keep + lane; e < width; e += 64) {
        list_ids[static_cast<size_t>(node) * width + e] = kInvalid;
        list_dists[static_cast<size_t>(node) * width + e] = FLT_MAX;
    }
    __builtin_amdgcn_wave_barrier();
    if (static_cast<uint32_t>(lane) < bloom_words) bloom[static_cast<size_t>(node) * bloom_words + lane] = filter[lane];
    if (lane == 0) {
        inbox_counts[node] = 0;
        counts[static_cast<size_t>(node) * 4 + 0] = total_new;
        counts[static_cast<size_t>(node) * 4 + 1] = total_old < kSamples ? total_old : kSamples;
        if (!rev_new) {   // with the scatter fused in, other wavefronts are adding to these two right now; the join clears them
            counts[static_cast<size_t>(node) * 4 + 2] = 0;
            counts[static_cast<size_t>(node) * 4 + 3] = 0;
        }
        if (stats) {   // striped over 1024 slots: one shared address would serialise every wavefront of the launch
            unsigned long long* slot = stats + 2 * (blockIdx.x & 1023u);
            atomicAdd(&slot[0], static_cast<unsigned long long>(raw));
            if (raw > inbox_cap) atomicAdd(&slot[1], static_cast<unsigned long long>(raw - inbox_cap));
        }
    }
}

template <int MMAX>
__global__ __launch_bounds__(256) void nnd_merge_kernel(uint32_t* list_ids, float* list_dists, uint32_t* inbox_counts, const uint2* inbox, uint32_t num,
                                                        uint32_t width, uint32_t inbox_cap, uint32_t* bloom, uint32_t bloom_sets, uint32_t* fwd_new,
                                                        uint32_t* fwd_old, uint32_t* counts, unsigned long long* stats, Segments segs, uint32_t* rev_new,
                                                        uint32_t* rev_old) {
    __shared__ uint32_t filter_lds[4][64];
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const uint32_t node = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (node >= num) return;
    uint32_t seg_start, seg_len;
    const uint32_t seg = locate_uniform(segs, node, seg_start, seg_len);
    if (segs.state[seg] == kDone) return;
    uint32_t* filter = filter_lds[wave];
    const uint32_t bloom_words = bloom_sets * 16;
    if (static_cast<uint32_t>(lane) < bloom_words) filter[lane] = bloom[static_cast<size_t>(node) * bloom_words + lane];
    const uint32_t raw = inbox_counts[node];
    const uint32_t held = width + (raw < inbox_cap ? raw : inbox_cap);   // the same for every lane of the wavefront
    if (held <= 64)
        merge_node<64>(list_ids, list_dists, inbox_counts, inbox, width, inbox_cap, bloom, bloom_sets, fwd_new, fwd_old, counts, stats, segs, node,
                       seg, raw, filter, lane, seg_start, rev_new, rev_old);
    else if (MMAX == 128 || held <= 128)
        merge_node<128>(list_ids, list_dists, inbox_counts, inbox, width, inbox_cap, bloom, bloom_sets, fwd_new, fwd_old, counts, stats, segs, node,
                        seg, raw, filter, lane, seg_start, rev_new, rev_old);
    else
        merge_node<256>(list_ids, list_dists, inbox_counts, inbox, width, inbox_cap, bloom, bloom_sets, fwd_new, fwd_old, counts, stats, segs, node,
                        seg, raw, filter, lane, seg_start, rev_new, rev_old);
}

// Termination test of GNND::build's update_and_sample (nn_descent.cuh:1270-1284): a partition whose sampled update
// count falls below termination_threshold * rows * dim / 100 (rows = all rows of the build, as in the reference) runs
// one more round -- the reference has already started that round's join when the host notices -- and then rests.
__global__ void nnd_converge_kernel(Segments segs, float limit) {
    const uint32_t s = blockIdx.x * blockDim.x + threadIdx.x;
    if (s >= segs.count) return;
    const uint32_t state = segs.state[s];
    if (state == kLastRound) {
        segs.state[s] = kDone;
    } else if (state == kActive && static_cast<float>(segs.updates[s]) < limit) {
        segs.state[s] = kLastRound;
    }
    segs.updates[s] = 0;
}

// ---- finalize (shrink step :1376-1402): first `degree` ids of each list; unfilled slots get a pseudo-random id
__host__ __device__ inline uint32_t xorshift32(uint32_t u) {   // reference utils.cuh:14-19
    u ^= u >> 13;
    u ^= u << 27;
    u ^= u >> 5;
    return u * 0x9E3779B9u;
}

__global__ __launch_bounds__(1024) void nnd_stats_reduce_kernel(const unsigned long long* striped, unsigned long long* out) {
    __shared__ unsigned long long part[2][1024];
    part[0][threadIdx.x] = striped[2 * threadIdx.x];
    part[1][threadIdx.x] = striped[2 * threadIdx.x + 1];
    __syncthreads();
    for (int off = 512; off > 0; off >>= 1) {
        if (static_cast<int>(threadIdx.x) < off) {
            part[0][threadIdx.x] += part[0][threadIdx.x + off];
            part[1][threadIdx.x] += part[1][threadIdx.x + off];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        out[0] = part[0][0];
        out[1] = part[1][0];
    }
}

__global__ __launch_bounds__(256) void nnd_finalize_kernel(const uint32_t* list_ids, uint32_t num, uint32_t width, uint32_t degree, Segments segs,
                                                           uint32_t* knn_graph) {
    const uint32_t idx = blockIdx.x * 256 + threadIdx.x;
    const uint32_t node = idx / degree, j = idx % degree;
    if (node >= num) return;
    uint32_t start, len;
    locate(segs, node, start, len);
    const uint32_t e = list_ids[static_cast<size_t>(node) * width + j];
    const uint32_t id = e & ~kOld;
    knn_graph[static_cast<size_t>(node) * degree + j] = (e != kInvalid && id < len) ? id : xorshift32(node * width + j) % (len ? len : 1);
}

}  // namespace glide

using namespace glide;

namespace {
uint32_t nnd_width(uint32_t degree) { return round_up32(static_cast<uint32_t>(degree * (degree <= 32 ? 1.0 : 1.3))); }  // nn_descent.cuh:1427-1428
uint32_t nnd_inbox_cap(uint32_t width) { return 256 - width; }   // list + inbox fill one 256-element sort
size_t align256(size_t x) { return (x + 255) / 256 * 256; }

struct NndLayout {
    size_t half_rows, norms, list_ids, list_dists, fwd_new, fwd_old, rev_new, rev_old, counts, inbox_counts, inbox, bloom, stats, seg_state, seg_updates, total;
    uint32_t width, cap, dim_pad, bloom_sets;
};
NndLayout nnd_layout(uint32_t num, uint32_t dim, uint32_t degree) {
    NndLayout l;
    l.width = nnd_width(degree);
    l.cap = nnd_inbox_cap(l.width);
    l.dim_pad = (dim + 7) / 8 * 8;
    l.bloom_sets = nnd_width(static_cast<uint32_t>(1.5 * degree)) / 32;   // internal degree / 32 (nn_descent.cuh:962, params.cuh:23-24)
    const size_t n = num;
    size_t off = 0;
    auto take = [&off](size_t bytes) { size_t o = off; off += align256(bytes); return o; };
    l.half_rows = take(n * l.dim_pad * 2);
    l.norms = take(n * 4);
    l.list_ids = take(n * l.width * 4);
    l.list_dists = take(n * l.width * 4);
    l.fwd_new = take(n * kSamples * 4);
    l.fwd_old = take(n * kSamples * 4);
    l.rev_new = take(n * kSamples * 4);
    l.rev_old = take(n * kSamples * 4);
    l.counts = take(n * 16);
    l.inbox_counts = take(n * 4);
    l.inbox = take(n * l.cap * 8);
    l.bloom = take(n * l.bloom_sets * 64);
    l.stats = take(1024 * 16);
    l.seg_state = take(kMaxSegments * 4);
    l.seg_updates = take(kMaxSegments * 4);
    l.total = off;
    return l;
}
}  // namespace

extern "C" {

size_t glide_hip_nnd_workspace_bytes(uint32_t reorder_num, uint32_t dim, uint32_t knn_degree) {
    return nnd_layout(reorder_num, dim, knn_degree).total;
}

namespace {
struct NndCtx {
    NndLayout l;
    _Float16* half_rows;
    float* norms;
    uint32_t* list_ids;
    float* list_dists;
    uint32_t *fwd_new, *fwd_old, *rev_new, *rev_old, *counts, *inbox_counts;
    uint2* inbox;
    uint32_t* bloom;
    unsigned long long* stats;
    Segments segs;
    uint32_t n;
    hipStream_t s;
};

int nnd_context(NndCtx& c, uint32_t reorder_num, uint32_t dim, const uint32_t* segment_starts, const uint32_t* segment_lengths,
                uint32_t segment_num, uint32_t knn_degree, void* workspace, size_t workspace_bytes, void* stream) {
    if (!segment_starts || !segment_lengths || !workspace) return GLIDE_ERR_BAD_ARGUMENT;
    if (dim == 0 || segment_num == 0 || knn_degree == 0 || reorder_num == 0) return GLIDE_ERR_BAD_ARGUMENT;
    if (segment_num > kMaxSegments) return GLIDE_ERR_UNSUPPORTED;
    if (nnd_width(knn_degree) > 96 || dim % 4 != 0) return GLIDE_ERR_UNSUPPORTED;   // also keeps the Bloom filter within 64 words
    // one thread per list slot / per sample: the products must fit the 32-bit launch arithmetic (44 M rows at width 96)
    if (static_cast<unsigned long long>(reorder_num) * nnd_width(knn_degree) >= 0xffffffffull || reorder_num >= (1u << 26)) return GLIDE_ERR_UNSUPPORTED;
    c.l = nnd_layout(reorder_num, dim, knn_degree);
    if (c.l.bloom_sets > 4) return GLIDE_ERR_UNSUPPORTED;
    if (workspace_bytes < c.l.total || reinterpret_cast<uintptr_t>(workspace) % 16) return GLIDE_ERR_BAD_ARGUMENT;
    unsigned char* w = static_cast<unsigned char*>(workspace);
    c.half_rows = reinterpret_cast<_Float16*>(w + c.l.half_rows);
    c.norms = reinterpret_cast<float*>(w + c.l.norms);
    c.list_ids = reinterpret_cast<uint32_t*>(w + c.l.list_ids);
    c.list_dists = reinterpret_cast<float*>(w + c.l.list_dists);
    c.fwd_new = reinterpret_cast<uint32_t*>(w + c.l.fwd_new);
    c.fwd_old = reinterpret_cast<uint32_t*>(w + c.l.fwd_old);
    c.rev_new = reinterpret_cast<uint32_t*>(w + c.l.rev_new);
    c.rev_old = reinterpret_cast<uint32_t*>(w + c.l.rev_old);
    c.counts = reinterpret_cast<uint32_t*>(w + c.l.counts);
    c.inbox_counts = reinterpret_cast<uint32_t*>(w + c.l.inbox_counts);
    c.inbox = reinterpret_cast<uint2*>(w + c.l.inbox);
    c.bloom = reinterpret_cast<uint32_t*>(w + c.l.bloom);
    c.stats = reinterpret_cast<unsigned long long*>(w + c.l.stats);
    c.segs = Segments{segment_starts, segment_lengths, segment_num, reinterpret_cast<uint32_t*>(w + c.l.seg_state),
                      reinterpret_cast<uint32_t*>(w + c.l.seg_updates)};
    c.n = reorder_num;
    c.s = as_stream(stream);
    return GLIDE_OK;
}

int nnd_prepare(const NndCtx& c, const float* data, uint32_t dim, uint32_t seed) {
    int rc = glide_hip_fill_u32(reinterpret_cast<uint32_t*>(c.stats), 0u, 1024 * 4, c.s);
    if (rc != GLIDE_OK) return rc;
    rc = glide_hip_fill_u32(c.bloom, 0u, static_cast<size_t>(c.n) * c.l.bloom_sets * 16, c.s);
    if (rc != GLIDE_OK) return rc;
    rc = glide_hip_fill_u32(c.segs.state, 0u, 2 * kMaxSegments, c.s);   // state and updates are adjacent
    if (rc != GLIDE_OK) return rc;
    hipLaunchKernelGGL(nnd_prepare_kernel, dim3(ceil_div(c.n, 4)), dim3(256), 0, c.s, data, c.n, dim, c.l.dim_pad, c.half_rows, c.norms);
    hipLaunchKernelGGL(nnd_init_kernel, dim3(ceil_div(c.n * c.l.width, 256)), dim3(256), 0, c.s, c.list_ids, c.list_dists, c.inbox_counts, c.n,
                       c.l.width, c.segs, seed);
    // first samples come from the random lists (sample_graph(true), nn_descent.cuh:1266); later ones from the merge
    hipLaunchKernelGGL(nnd_sample_kernel, dim3(ceil_div(c.n, 4)), dim3(256), 0, c.s, c.list_ids, c.n, c.l.width, c.segs, c.fwd_new, c.fwd_old, c.counts);
    return launch_status();
}

int nnd_reverse(const NndCtx& c) {
    hipLaunchKernelGGL(nnd_reverse_kernel, dim3(ceil_div(c.n * 64, 256)), dim3(256), 0, c.s, c.fwd_new, c.fwd_old, c.counts, c.rev_new, c.rev_old, c.n,
                       c.segs);
    return launch_status();
}

int nnd_join(const NndCtx& c) {
    GLIDE_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(&nnd_join_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      static_cast<int>(sizeof(JoinLds))));
    JoinArgs ja{c.half_rows, c.norms, c.fwd_new, c.fwd_old, c.rev_new, c.rev_old, c.counts, c.inbox_counts, c.inbox, c.stats,
                c.n, c.l.dim_pad, c.l.width, c.l.cap, c.segs};
    hipLaunchKernelGGL(nnd_join_kernel, dim3(c.n), dim3(256), sizeof(JoinLds), c.s, ja);
    return launch_status();
}

// scatter_reverse: the new and old samples a node draws are appended to the reverse lists of their targets right away
// (what the next round's nnd_reverse would do), while the sort of other nodes keeps the vector ALU busy
int nnd_merge(const NndCtx& c, bool with_stats, bool scatter_reverse = false) {
    unsigned long long* stats = with_stats ? c.stats : nullptr;
    uint32_t* rev_new = scatter_reverse ? c.rev_new : nullptr;
    uint32_t* rev_old = scatter_reverse ? c.rev_old : nullptr;
    const uint32_t m = c.l.width + c.l.cap;
    if (m <= 128) {
        hipLaunchKernelGGL(nnd_merge_kernel<128>, dim3(ceil_div(c.n, 4)), dim3(256), 0, c.s, c.list_ids, c.list_dists, c.inbox_counts, c.inbox, c.n,
                           c.l.width, c.l.cap, c.bloom, c.l.bloom_sets, c.fwd_new, c.fwd_old, c.counts, stats, c.segs, rev_new, rev_old);
    } else {
        hipLaunchKernelGGL(nnd_merge_kernel<256>, dim3(ceil_div(c.n, 4)), dim3(256), 0, c.s, c.list_ids, c.list_dists, c.inbox_counts, c.inbox, c.n,
                           c.l.width, c.l.cap, c.bloom, c.l.bloom_sets, c.fwd_new, c.fwd_old, c.counts, stats, c.segs, rev_new, rev_old);
    }
    return launch_status();
}

int nnd_converge(const NndCtx& c, uint32_t dim, float termination_threshold) {
    // update_counter < termination_threshold * nrow * dim / counter_interval (nn_descent.cuh:1280), evaluated in float
    const float limit = termination_threshold * static_cast<float>(c.n) * static_cast<float>(dim) / static_cast<float>(kCounterInterval);
    hipLaunchKernelGGL(nnd_converge_kernel, dim3(ceil_div(c.segs.count, 256)), dim3(256), 0, c.s, c.segs, limit);
    return launch_status();
}

int nnd_finalize(const NndCtx& c, uint32_t knn_degree, uint32_t* knn_graph, unsigned long long* stats_out) {
    hipLaunchKernelGGL(nnd_finalize_kernel, dim3(ceil_div(c.n * knn_degree, 256)), dim3(256), 0, c.s, c.list_ids, c.n, c.l.width, knn_degree, c.segs,
                       knn_graph);
    if (stats_out) hipLaunchKernelGGL(nnd_stats_reduce_kernel, dim3(1), dim3(1024), 0, c.s, c.stats, stats_out);
    return launch_status();
}
}  // namespace

int glide_hip_nnd_build(const float* reorder_data, uint32_t reorder_num, uint32_t dim, const uint32_t* segment_starts,
                        const uint32_t* segment_lengths, uint32_t segment_num, uint32_t knn_degree, uint32_t iterations,
                        float termination_threshold, uint32_t seed, uint32_t* knn_graph, void* workspace, size_t workspace_bytes,
                        unsigned long long* stats_out, void* stream) {
    if (!reorder_data || !knn_graph || !(termination_threshold >= 0.f)) return GLIDE_ERR_BAD_ARGUMENT;
    if (reorder_num == 0 && segment_starts && segment_lengths && workspace && dim && segment_num && knn_degree) return GLIDE_OK;
    NndCtx c;
    int rc = nnd_context(c, reorder_num, dim, segment_starts, segment_lengths, segment_num, knn_degree, workspace, workspace_bytes, stream);
    if (rc != GLIDE_OK) return rc;
    if ((rc = nnd_prepare(c, reorder_data, dim, seed)) != GLIDE_OK) return rc;
    for (uint32_t it = 0; it < iterations; it++) {
        if (it == 0 && (rc = nnd_reverse(c)) != GLIDE_OK) return rc;   // later rounds: the merge of the round before has done it
        if ((rc = nnd_join(c)) != GLIDE_OK) return rc;
        if ((rc = nnd_merge(c, stats_out != nullptr, it + 1 < iterations)) != GLIDE_OK) return rc;
        if ((rc = nnd_converge(c, dim, termination_threshold)) != GLIDE_OK) return rc;
        // GNND::build leaves its loop when the update count falls below the limit (nn_descent.cuh:1270-1284).  Here the
        // partitions rest one by one on the device; once none is active the remaining rounds would only launch kernels
        // that return at once, so the states are read back (a few hundred bytes) and the loop ends.
        if (termination_threshold > 0.f && it >= 2 && it + 1 < iterations) {
            std::vector<uint32_t> states(segment_num);
            GLIDE_HIP_TRY(hipMemcpyAsync(states.data(), c.segs.state, sizeof(uint32_t) * segment_num, hipMemcpyDeviceToHost, c.s));
            GLIDE_HIP_TRY(hipStreamSynchronize(c.s));
            bool any_active = false;
            for (uint32_t st : states) any_active |= st != kDone;
            if (!any_active) break;
        }
    }
    return nnd_finalize(c, knn_degree, knn_graph, stats_out);
}

int glide_hip_nnd_layout(uint32_t reorder_num, uint32_t dim, uint32_t knn_degree, glide_nnd_layout* out) {
    if (!out || dim == 0 || knn_degree == 0) return GLIDE_ERR_BAD_ARGUMENT;
    if (nnd_width(knn_degree) > 96 || dim % 4 != 0) return GLIDE_ERR_UNSUPPORTED;
    const NndLayout l = nnd_layout(reorder_num, dim, knn_degree);
    out->half_rows = l.half_rows; out->norms = l.norms; out->list_ids = l.list_ids; out->list_dists = l.list_dists;
    out->fwd_new = l.fwd_new; out->fwd_old = l.fwd_old; out->rev_new = l.rev_new; out->rev_old = l.rev_old;
    out->counts = l.counts; out->inbox_counts = l.inbox_counts; out->inbox = l.inbox; out->bloom = l.bloom;
    out->segment_state = l.seg_state; out->segment_updates = l.seg_updates; out->total = l.total;
    out->width = l.width; out->inbox_cap = l.cap; out->row_halfs = l.dim_pad; out->bloom_sets = l.bloom_sets;
    return GLIDE_OK;
}

int glide_hip_nnd_prepare(const float* reorder_data, uint32_t reorder_num, uint32_t dim, const uint32_t* segment_starts,
                          const uint32_t* segment_lengths, uint32_t segment_num, uint32_t knn_degree, uint32_t seed, void* workspace,
                          size_t workspace_bytes, void* stream) {
    if (!reorder_data) return GLIDE_ERR_BAD_ARGUMENT;
    NndCtx c;
    int rc = nnd_context(c, reorder_num, dim, segment_starts, segment_lengths, segment_num, knn_degree, workspace, workspace_bytes, stream);
    return rc != GLIDE_OK ? rc : nnd_prepare(c, reorder_data, dim, seed);
}

int glide_hip_nnd_reverse_sample(uint32_t reorder_num, uint32_t dim, const uint32_t* segment_starts, const uint32_t* segment_lengths,
                                 uint32_t segment_num, uint32_t knn_degree, void* workspace, size_t workspace_bytes, void* stream) {
    NndCtx c;
    int rc = nnd_context(c, reorder_num, dim, segment_starts, segment_lengths, segment_num, knn_degree, workspace, workspace_bytes, stream);
    return rc != GLIDE_OK ? rc : nnd_reverse(c);
}

int glide_hip_nnd_local_join(uint32_t reorder_num, uint32_t dim, const uint32_t* segment_starts, const uint32_t* segment_lengths,
                             uint32_t segment_num, uint32_t knn_degree, void* workspace, size_t workspace_bytes, void* stream) {
    NndCtx c;
    int rc = nnd_context(c, reorder_num, dim, segment_starts, segment_lengths, segment_num, knn_degree, workspace, workspace_bytes, stream);
    return rc != GLIDE_OK ? rc : nnd_join(c);
}

int glide_hip_nnd_merge(uint32_t reorder_num, uint32_t dim, const uint32_t* segment_starts, const uint32_t* segment_lengths,
                        uint32_t segment_num, uint32_t knn_degree, void* workspace, size_t workspace_bytes, void* stream) {
    NndCtx c;
    int rc = nnd_context(c, reorder_num, dim, segment_starts, segment_lengths, segment_num, knn_degree, workspace, workspace_bytes, stream);
    return rc != GLIDE_OK ? rc : nnd_merge(c, true);
}

int glide_hip_nnd_converge(uint32_t reorder_num, uint32_t dim, const uint32_t* segment_starts, const uint32_t* segment_lengths,
                           uint32_t segment_num, uint32_t knn_degree, float termination_threshold, void* workspace, size_t workspace_bytes,
                           void* stream) {
    if (!(termination_threshold >= 0.f)) return GLIDE_ERR_BAD_ARGUMENT;
    NndCtx c;
    int rc = nnd_context(c, reorder_num, dim, segment_starts, segment_lengths, segment_num, knn_degree, workspace, workspace_bytes, stream);
    return rc != GLIDE_OK ? rc : nnd_converge(c, dim, termination_threshold);
}

int glide_hip_nnd_finalize(uint32_t reorder_num, uint32_t dim, const uint32_t* segment_starts, const uint32_t* segment_lengths,
                           uint32_t segment_num, uint32_t knn_degree, uint32_t* knn_graph, unsigned long long* stats_out, void* workspace,
                           size_t workspace_bytes, void* stream) {
    if (!knn_graph) return GLIDE_ERR_BAD_ARGUMENT;
    NndCtx c;
    int rc = nnd_context(c, reorder_num, dim, segment_starts, segment_lengths, segment_num, knn_degree, workspace, workspace_bytes, stream);
    return rc != GLIDE_OK ? rc : nnd_finalize(c, knn_degree, knn_graph, stats_out);
}

}  // extern "C"
