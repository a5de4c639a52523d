// NN-descent kNN-graph construction, entirely on the device.
//
// Reference: nn_descent.cuh -- preprocess_data_kernel (:445-488), sampling on the host (GnndGraph::sample_graph
// :1040-1071, sample_graph_new :973-1001), add_rev_edges_kernel (:490-507), local_join_kernel (:668-914),
// insert_to_global_graph (:509-579), host merge update_graph (:1106-1126) and the shrink step (:1376-1402).
//
// What is kept: fp16 rows with fp32 squared norms, <= 32 new + <= 32 old forward samples per node, reverse
// samples capped at 32, a 64 x 64 distance tile per phase (new x new, new x old) computed on the matrix cores
// with the norm-trick epilogue, and one offer per row / column (its nearest partner) per phase.
// What is different: the kNN lists, flags, Bloom filters and samples never leave HBM.  An offer is a pair of 64-bit
// atomic minima on two slots of its target's table (no locks, nothing returned); reverse samples go to plain per-node lists with
// an overflow table that keeps the smallest sources.  What a node holds at the end of a round -- all that the
// reference's 32-wide device list and its 32 reverse samples would be drawn from -- is the same whatever the order of
// arrival, so a build is reproducible.  A merge kernel then applies the reference's rules: of a node's offers the
// best 32 count, those not yet listed enter the sub-list id % num_sub (each sub-list keeps its 32 nearest), those the
// Bloom filter has not seen are the next "new" samples.  All ids are partition-local.
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
__device__ __forceinline__ uint32_t locate_uniform(const Segments& s, uint32_t node, uint32_t& start, uint32_t& len, uint32_t* state = nullptr) {
    for (uint32_t base = 0; base < s.count; base += 64) {
        const uint32_t i = base + lane_id();
        const bool in_range = i < s.count;
        const uint32_t st = in_range ? s.starts[i] : 0u, ln = in_range ? s.lengths[i] : 0u;
        const uint32_t state_i = state && in_range ? s.state[i] : 0u;
        // the last segment takes whatever lies beyond it, as the scalar search does
        const uint64_t m = ballot(in_range && (node < st + ln || i + 1 == s.count));
        if (m) {
            const int at = __ffsll(static_cast<long long>(m)) - 1;   // the values come from the lane that tested the segment
            start = read_lane(st, at);
            len = read_lane(ln, at);
            if (state) *state = read_lane(state_i, at);
            return base + at;
        }
    }
    start = len = 0;   // no segments at all: not reached, the entry points refuse segment_num == 0
    if (state) *state = kDone;
    return 0;
}

// ---- prepare: fp32 rows -> fp16 rows (stride dim_pad, zero padded) + squared norms of the fp32 input
__global__ __launch_bounds__(256) void nnd_prepare_kernel(const float* data, uint32_t num, uint32_t dim, uint32_t dim_pad, _Float16* half_rows,
                                                          float2* norms /* squared norm; offer threshold (none yet) */) {
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
    if (lane == 0) norms[i] = make_float2(acc, __uint_as_float(kInvalid));
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

__global__ __launch_bounds__(256) void nnd_init_kernel(uint32_t* list_ids, float* list_dists, uint32_t num, uint32_t width,
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
}

// ---- sampling: first <= 32 new entries (marked old afterwards) and first <= 32 entries that were already old.
// The list is stored column-major over its sub-lists (slot = rank * num_sub + sub), so storage order is the order in
// which the reference scans it (sample_graph :1052-1068).
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

// ---- where reverse samples arrive -----------------------------------------------------------------------------------
// They go first to a plain list of the receiving node: one atomic add reserves a slot, a store fills it.  As long as
// a list does not fill up it holds every arrival, so the set it ends up with does not depend on the order of arrival;
// the consumer sorts it.  What arrives after a list is full goes to the node's overflow table, which keeps the
// smallest keys whatever the order of arrival:
//   a table is made of buckets of 16 words, 15 slots and, last, the bucket's bound = the smallest key it has turned
//   away (all ones: none yet); a key's bucket and first slot are hashes of its id.  A slot keeps the smaller of the key
//   it holds and the key that arrives (one atomic minimum); the larger one goes on to the next slot of the bucket.
//   Slot contents only ever decrease, so a key that has passed all 15 slots is larger than everything the bucket holds
//   in the end and is dropped: a bucket ends with the 15 smallest distinct keys sent to it.  A key that is not smaller
//   than the bound need not look further, which keeps a node that receives thousands of keys cheap.
// The join only uses the smallest 32 sources of list + table (the reference's 32 reverse samples).  One of those could
// only be missing if 15 smaller keys shared its bucket, i.e. if 16 of a node's 32 smallest keys fell into one of 16
// buckets: with the smallest 32 of every node intact, the result is the same on every run.
// A node that receives thousands of keys round after round would make every sender wait for atomics on the same few
// cache lines.  Such a node therefore announces a threshold for the next round, read by the senders before anything
// else (a plain read of a read-only array): when its list overflowed, the 56th smallest source of this round -- like
// the smallest 32, the smallest 56 of list + table do not depend on the order of arrival.  Sources that are not below
// the threshold stay away.  As long as at least 32 sources below it arrive, the smallest 32 are what they would have
// been without it; the threshold is kept while arrivals stay plentiful and withdrawn when they do not.  Nodes that are
// offered thousands of candidates announce a distance threshold in the same way (kOfferCrowded below).
constexpr uint32_t kBucketWords = 16, kBucketData = 15;
constexpr uint32_t kRevCap = 64;         // reverse samples per node, kind and round before the overflow table takes over
// Row stride of the reverse lists, in entries.  Arrivals fill a row from its start, so with a power-of-two stride
// (256 B) the busy front parts of all rows would sit on the same few memory channels.
constexpr uint32_t kRevStride = kRevCap + 8;
// Offers of a round: per node a table of (distance bits : candidate id) keys, 256 slots for lists of one sub-list, 512
// for lists of several.  An offer goes to two slots of one 16-slot (128-byte) line of its target's table, both chosen
// by hashes of the candidate's id, and stays in each if it is the smallest key that slot has seen this round (64-bit
// atomic minima without a return value).  Copies of one offer, found by several joins, are the same key and fall
// together; two different candidates in one slot leave the nearer one, and an offer is lost only if both its slots
// hold nearer candidates (about one of a node's best 32 in ten rounds; with a single slot it was two a round, which
// showed as a lag of 1.4 points of graph recall in the first rounds).  What the table holds at the end of the round
// does not depend on the order of arrival.
constexpr uint32_t kOfferSlotsNarrow = 256, kOfferSlotsWide = 512;   // lists of one sub-list; of several (SLOTS below)
__host__ __device__ constexpr uint32_t offer_slots_for(uint32_t width) { return width > 32 ? kOfferSlotsWide : kOfferSlotsNarrow; }
constexpr uint32_t kRevSlots = 256;      // overflow table per node and kind: 16 buckets of source ids
constexpr unsigned long long kNoOffer = ~0ull;
constexpr uint32_t kOfferCrowdedEighths = 5;   // a node whose table is this full (in eighths) announces a threshold: ...
constexpr uint32_t kOfferThrRank = 64;    // ... the distance of its 64th best offer
constexpr uint32_t kOfferKeepHeld = 40;   // a threshold in force is withdrawn when fewer offers than this are held
constexpr uint32_t kRevThrRank = 56;      // the threshold of a node whose reverse list overflowed: its 56th smallest source
constexpr uint32_t kRevKeepArrivals = 40; // fewer arrivals than this withdraw it

__device__ __forceinline__ uint32_t id_hash(uint32_t id) { return id * 0x9E3779B1u; }
__device__ __forceinline__ uint32_t first_slot(uint32_t hash) { return __umulhi(hash * 0x85EBCA6Bu, kBucketData); }   // 0..14
// Slot of a candidate in an offer table.  The salt changes with the round, so two candidates that share a slot in one
// round do not share it in the next.
__device__ __forceinline__ uint32_t offer_slot(uint32_t cand, uint32_t salt, uint32_t shift) { return id_hash(cand ^ salt) >> shift; }
// the second slot in the 16-slot (128-byte) line of the first: another of its 15 positions
__device__ __forceinline__ uint32_t offer_slot_beside(uint32_t first, uint32_t cand, uint32_t salt) {
    return (first & ~15u) | ((first + 1u + __umulhi((cand ^ salt) * 0xC2B2AE35u, 15u)) & 15u);
}
__device__ __forceinline__ uint32_t round_salt(uint32_t round) { return round * 0x85EBCA6Bu; }

// One source id into a reverse overflow table (256 words).  The bound is read first: a table only comes into play for
// nodes with many arrivals, and once its buckets are full nearly every further arrival ends here after one read.
__device__ __forceinline__ void reverse_insert(uint32_t* table, uint32_t key) {
    const uint32_t h = id_hash(key);
    uint32_t* b = table + (h >> 28) * kBucketWords;
    if (key >= __hip_atomic_load(&b[kBucketData], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) return;
    uint32_t pos = first_slot(h);
    for (uint32_t probe = 0; probe < kBucketData; probe++) {
        const uint32_t old = atomicMin(&b[pos], key);
        if (old == kInvalid || old == key) return;   // settled in an empty slot, or already there
        if (old > key) key = old;                    // the displaced key carries on
        pos = pos + 1 == kBucketData ? 0 : pos + 1;
    }
    atomicMin(&b[kBucketData], key);   // larger than all 15 the bucket holds
}

// add_rev_edges_kernel (:490-507) for one sample: list `source` appends itself to the reverse list of `target` (both
// row indices of the whole build; `source_local` is what is stored).  The reference keeps the first 32 arrivals; here
// the 32 smallest sources count, which is what a sweep over the lists in order keeps.
__device__ __forceinline__ void reverse_append(uint32_t* counts, uint32_t* rev_list, uint32_t* rev_tables, const uint32_t* rev_thr, size_t target,
                                               uint32_t which, uint32_t source_local) {
    if (source_local >= rev_thr[target * 2 + which]) return;   // the target has asked sources from here on to stay away
    const uint32_t pos = atomicAdd(&counts[target * 4 + 2 + which], 1u);
    if (pos < kRevCap)
        rev_list[target * kRevStride + pos] = source_local;
    else
        reverse_insert(rev_tables + (target * 2 + which) * kRevSlots, source_local);
}

// ---- reverse samples as a stage of its own: every list enters the reverse tables of its samples
__global__ __launch_bounds__(256) void nnd_reverse_kernel(const uint32_t* fwd_new, const uint32_t* fwd_old, uint32_t* counts, uint32_t* rev_new,
                                                          uint32_t* rev_old, uint32_t* rev_tables, const uint32_t* rev_thr, uint32_t num, Segments segs) {
    const uint32_t idx = blockIdx.x * 256 + threadIdx.x;
    const uint32_t node = idx / 64, j = idx % 64;
    if (node >= num) return;
    uint32_t start, len;
    uint32_t state;
    locate_uniform(segs, node, start, len, &state);
    if (state == kDone) return;
    const uint32_t which = j / kSamples, k = j % kSamples;   // 0: new, 1: old
    if (k >= counts[static_cast<size_t>(node) * 4 + which]) return;
    const uint32_t v = (which ? fwd_old : fwd_new)[static_cast<size_t>(node) * kSamples + k];
    reverse_append(counts, which ? rev_old : rev_new, rev_tables, rev_thr, static_cast<size_t>(start) + v, which, node - start);
}

// ---- local join ---------------------------------------------------------------------------------------------
struct JoinArgs {
    const _Float16* half_rows;
    const float2* norms;           // num x (squared norm, offer threshold: offers whose distance bits are not below it stay away; all ones: none)
    const uint32_t* fwd_new;
    const uint32_t* fwd_old;
    const uint32_t* rev_new;       // num x kRevCap: the first reverse samples to arrive
    const uint32_t* rev_old;
    uint32_t* rev_tables;          // num x 2 x kRevSlots: where later arrivals went; emptied by the join that reads them
    uint32_t* rev_thr;             // num x 2: sources not below it stay away in the next scatter (all ones: none)
    uint32_t* counts;              // num x 4: forward new / old, reverse new / old arrivals (restarted by the members kernel)
    uint32_t* members;             // num x 128: the lists a join works on, new members first (64 slots), then old ones
    uint32_t* member_counts;       // num x 2: how many new and old members
    unsigned long long* offers;    // num x offer_slots: the offer tables
    uint32_t offer_slots, slot_shift;   // slot_shift = 32 - log2(offer_slots)
    const uint32_t* round;         // rounds completed so far (salt of the slot hash)
    unsigned long long* stats;     // striped: [1] offers that stayed away because of their target's threshold (nullable)
    uint32_t num, dim_pad;
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
    __attribute__((aligned(16))) uint32_t new_ids[kBi], old_ids[kBi];   // read four at a time
    __attribute__((aligned(16))) float new_norms[kBi], old_norms[kBi];
    uint32_t new_thr[kBi], old_thr[kBi];                           // offer thresholds of the members
    float part_d[2][2 * kBi];      // column arg-mins of the two row blocks: [new x new | new x old][row block * 64 + column]
    uint32_t part_i[2][2 * kBi];
};

struct MembersLds {   // per wavefront = per list; the two kinds of sample use it one after the other
    __attribute__((aligned(16))) uint32_t rev_raw[4][kRevCap + kRevSlots];   // reverse samples as read: the list, then the overflow table
    uint32_t rev_sel[4][kSamples];                                 // their 32 smallest entries, ascending
    uint32_t rev_next_thr[4];
    uint32_t hash[4][128];
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

// Row (of a pass of 32) that thread `tid` of the workgroup stages: groups of 8 lanes 0, 1, 2, 3 ... take rows 0, 8, 1, 9 ...
__device__ __forceinline__ uint32_t staged_row(int tid) {
    const uint32_t g = static_cast<uint32_t>(tid) >> 3;
    return ((g & 1u) << 3) | ((g >> 1) & 7u) | (g & 16u);
}

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

// ---- who takes part in a join: one wavefront per list, ahead of the join proper.
// The members of a list are its forward samples and the 32 smallest sources of its reverse arrivals, duplicates
// removed (reference: sort + binary search, :625-666; forward samples first, so a point that is in both keeps its
// forward position).  This is light work on scattered reads: a kernel of its own runs it with eight wavefronts per
// SIMD, where the join, held to six workgroups per CU by its tiles, spent a third of its time on it.
__global__ __launch_bounds__(256) void nnd_members_kernel(JoinArgs a) {
    __shared__ MembersLds L;
    const int lane = lane_id(), wave = threadIdx.x >> 6;
    const uint32_t node = blockIdx.x * 4 + wave;
    if (node >= a.num) return;
    // everything is asked for before anything is known about it (one memory round trip): both reverse lists, the
    // forward samples (new ones in lanes 0..31, old ones in lanes 32..63), thresholds and counts
    const uint32_t rev_in[2] = {a.rev_new[static_cast<size_t>(node) * kRevStride + lane], a.rev_old[static_cast<size_t>(node) * kRevStride + lane]};
    const uint32_t forward_both = (lane < static_cast<int>(kSamples) ? a.fwd_new : a.fwd_old)[static_cast<size_t>(node) * kSamples + (lane & 31)];
    const uint2 thr_both = *reinterpret_cast<const uint2*>(a.rev_thr + static_cast<size_t>(node) * 2);
    const uint4 c4 = *reinterpret_cast<const uint4*>(a.counts + static_cast<size_t>(node) * 4);
    uint32_t seg_start, seg_len, state;
    locate_uniform(a.segs, node, seg_start, seg_len, &state);
    if (state == kDone) return;
    uint32_t* const raw = L.rev_raw[wave];
    uint32_t* const sel = L.rev_sel[wave];
    uint32_t* const set = L.hash[wave];
#pragma unroll
    for (int kind = 0; kind < 2; kind++) {   // 0: new, 1: old
        const bool is_old = kind != 0;
        uint32_t my_id = rev_in[kind];
        const uint32_t thr_in_force = is_old ? thr_both.y : thr_both.x;
        const uint32_t forward = static_cast<uint32_t>(__shfl(static_cast<int>(forward_both), (lane & 31) + 32 * kind));
        __builtin_amdgcn_wave_barrier();   // the kind before is done with the scratch
        set[lane] = kInvalid;
        set[lane + 64] = kInvalid;

        // Reverse samples: the 32 smallest sources that arrived, in ascending order.  Up to 64 arrivals sit in the list;
        // a node that received more also has an overflow table, which is read and emptied (bounds included) here.
        const uint32_t arrived = is_old ? c4.w : c4.z;
        if (static_cast<uint32_t>(lane) >= arrived) my_id = kInvalid;
        uint4 more = make_uint4(kInvalid, kInvalid, kInvalid, kInvalid);
        const bool overflowed = arrived > kRevCap;
        if (overflowed) {
            uint4* const quad = reinterpret_cast<uint4*>(a.rev_tables + (static_cast<size_t>(node) * 2 + kind) * kRevSlots) + lane;
            more = *quad;
            if ((more.x & more.y & more.z & more.w) != kInvalid) *quad = make_uint4(kInvalid, kInvalid, kInvalid, kInvalid);
            if ((lane & 3) == 3) more.w = kInvalid;   // word 15 of a bucket is its bound
            *reinterpret_cast<uint4*>(&raw[kRevCap + 4 * lane]) = more;
        }
        raw[lane] = my_id;
        if (lane < static_cast<int>(kSamples)) sel[lane] = kInvalid;
        if (lane == 0) L.rev_next_thr[wave] = kInvalid;
        __builtin_amdgcn_wave_barrier();
        if (!overflowed) {
            uint32_t rank = 0;
            // four slots a step, as far as the arrivals go (the slots behind them hold 0xffffffff and count for nothing)
            for (uint32_t j = 0; j < arrived; j += 4) {
                const uint4 q = *reinterpret_cast<const uint4*>(&raw[j]);
                rank += (q.x < my_id) + (q.y < my_id) + (q.z < my_id) + (q.w < my_id);
            }
            if (my_id != kInvalid && rank < kSamples) sel[rank] = my_id;
        } else {
            const uint32_t mine[5] = {my_id, more.x, more.y, more.z, more.w};
            uint32_t rank[5] = {0, 0, 0, 0, 0};
            for (uint32_t j = 0; j < kRevCap + kRevSlots; j += 4) {
                const uint4 q = *reinterpret_cast<const uint4*>(&raw[j]);
#pragma unroll
                for (int m = 0; m < 5; m++) rank[m] += (q.x < mine[m]) + (q.y < mine[m]) + (q.z < mine[m]) + (q.w < mine[m]);
            }
#pragma unroll
            for (int m = 0; m < 5; m++) {
                if (mine[m] != kInvalid && rank[m] < kSamples) sel[rank[m]] = mine[m];
                // after an overflow the 56th smallest source becomes the threshold of the scatter that follows: some 55
                // sources are then expected, few enough to stay in the list, enough for the smallest 32 to be complete
                if (mine[m] != kInvalid && rank[m] == kRevThrRank - 1) L.rev_next_thr[wave] = mine[m];
            }
        }
        __builtin_amdgcn_wave_barrier();
        if (lane == 0) {
            // a threshold that is in force stays while at least 40 sources still arrive
            const uint32_t next = overflowed ? L.rev_next_thr[wave] : (arrived >= kRevKeepArrivals ? thr_in_force : kInvalid);
            if (next != thr_in_force) a.rev_thr[static_cast<size_t>(node) * 2 + kind] = next;
            // this list's reverse samples are consumed here and now: the count restarts for the scatter that follows the join
            a.counts[static_cast<size_t>(node) * 4 + 2 + kind] = 0u;
        }
        // Forward samples (lanes 0..31) enter the set first, then the reverse ones (lanes 32..63).
        const uint32_t k = lane;
        const uint32_t id = k < kSamples ? (k < (is_old ? c4.y : c4.x) ? forward : kInvalid) : sel[k - kSamples];
        const bool usable = id != kInvalid && id < seg_len;
        bool keep = false;
        if (k < kSamples) keep = usable && lds_set_insert(set, id);
        __builtin_amdgcn_wave_barrier();
        if (k >= kSamples) keep = usable && lds_set_insert(set, id);
        const uint64_t m = ballot(keep);
        if (keep) a.members[static_cast<size_t>(node) * (2 * kBi) + kBi * kind + prefix_count(m)] = id;
        if (lane == 0) a.member_counts[static_cast<size_t>(node) * 2 + kind] = __popcll(m);
    }
}

// The join of one list by a workgroup of four wavefronts.  `lists`: which lists are the caller's.  kAllLists: every
// one; kWideLists: those with more than 32 new members, the others being nnd_join_narrow_kernel's.
constexpr int kAllLists = 0, kWideLists = 1;
__device__ __forceinline__ void join_list(const JoinArgs& a, JoinLds& L, const uint32_t node, const int lists) {
    const int tid = threadIdx.x, lane = lane_id(), wave = tid >> 6;
    // member ids are fetched before their counts are known (one memory round trip instead of two); slots beyond a
    // list hold what an earlier round left there, and count for nothing: their norm below is infinite
    const uint32_t member = tid < static_cast<int>(2 * kBi) ? a.members[static_cast<size_t>(node) * (2 * kBi) + tid] : kInvalid;
    const uint2 mc = *reinterpret_cast<const uint2*>(a.member_counts + static_cast<size_t>(node) * 2);
    uint32_t seg_start, seg_len;
    uint32_t state;
    locate_uniform(a.segs, node, seg_start, seg_len, &state);
    if (state == kDone) return;
    const uint32_t n_new = mc.x, n_old = mc.y;
    if (n_new == 0 || (lists != kAllLists && n_new <= kSamples)) return;
    if (tid < static_cast<int>(2 * kBi)) {
        (tid < static_cast<int>(kBi) ? L.new_ids : L.old_ids)[tid & 63] = member;
        (tid < static_cast<int>(kBi) ? L.new_norms : L.old_norms)[tid & 63] = __builtin_inff();   // replaced below for the rows the lists hold
    }
    __syncthreads();

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
    // rows, then old rows).  The two rows that 16 adjacent lanes store together are eight apart: with the row stride of
    // 36 words they then fall on opposite halves of the 64 banks (adjacent rows would overlap by four banks).  The loads of chunk k+1 are issued before the matrix instructions of chunk k.  Short chunks
    // keep the workgroup at 20 KB of LDS, so six of them share a CU instead of four.
    float4 pre[4];
    // Norm and offer threshold of a row are asked for with its first chunk and stored with it (a store right behind the
    // load would make the wavefront wait for every pass in turn).  Lane q of a row's group takes pass q, so a lane
    // holds one pair.
    float2 pre_norm = make_float2(0.f, 0.f);
    auto prefetch = [&](uint32_t k0) {
#pragma unroll
        for (int pass = 0; pass < 4; pass++) {
            const uint32_t r = pass * 32 + staged_row(tid), q = tid & 7;
            const bool old_row = r >= 64;
            const uint32_t rr = r & 63;
            const uint32_t d0 = k0 + q * 8;
            pre[pass] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (rr < (old_row ? n_old : n_new)) {
                const uint32_t id = (old_row ? L.old_ids : L.new_ids)[rr];
                if (d0 < a.dim_pad) pre[pass] = *reinterpret_cast<const float4*>(a.half_rows + static_cast<size_t>(seg_start + id) * a.dim_pad + d0);
                if (k0 == 0 && q == static_cast<uint32_t>(pass)) pre_norm = a.norms[seg_start + id];   // same round trip as the row
            }
        }
    };
    prefetch(0);
    for (uint32_t k0 = 0; k0 < a.dim_pad; k0 += kJoinChunk) {
        if (k0) __syncthreads();   // every wave is done with the previous chunk
#pragma unroll
        for (int pass = 0; pass < 4; pass++) {
            const uint32_t r = pass * 32 + staged_row(tid), q = tid & 7;
            *reinterpret_cast<float4*>(&(r >= 64 ? L.rows.xo : L.rows.xn)[r & 63][q * 8]) = pre[pass];
            if (k0 == 0 && q == static_cast<uint32_t>(pass) && (r & 63) < (r >= 64 ? n_old : n_new)) {
                (r >= 64 ? L.old_norms : L.new_norms)[r & 63] = pre_norm.x;
                (r >= 64 ? L.old_thr : L.new_thr)[r & 63] = __float_as_uint(pre_norm.y);
            }
        }
        __syncthreads();
        if (k0 + kJoinChunk < a.dim_pad) prefetch(k0 + kJoinChunk);
        if (need_nn) mfma_chunk(acc_nn, L.rows.xn, L.rows.xn, rb, cb, lane);
        if (need_no) mfma_chunk(acc_no, L.rows.xn, L.rows.xo, rb, cb, lane);
    }

    const int t = lane & 31, kh = lane >> 5;
    const uint32_t line = tid >> 2, part = tid & 3;
    // An offer is two atomic minima on slots of one line of the target's table; nothing comes back, so the wave does not
    // wait.  Two adjacent lanes take the two slots in one instruction: the chip carries out some 27 G scattered atomic
    // operations a second, and nearly twice as many when adjacent lanes aim at one 128-byte line.
    const uint32_t salt = round_salt(*a.round);
    uint32_t declined = 0;
    // A slot is read before anything is sent to it (the reads of a thread's two offers are under way while the row scan
    // runs): within a round a slot only ever gets smaller, so a minimum that would not get below what the read has found
    // changes nothing and is left out.  In the first rounds, where the wide lists are, that is every second one.
    struct Offer {
        unsigned long long* where;
        unsigned long long what, there;
    };
    auto address = [&](uint32_t target, uint32_t cand, float dist, uint32_t thr, bool second_slot) {
        Offer o{nullptr, 0, 0};
        if (cand == kInvalid || cand == target || cand >= seg_len || !(dist < FLT_MAX)) return o;
        if (__float_as_uint(dist) >= thr) {   // the target has asked offers from this distance on to stay away
            declined += !second_slot;
            return o;
        }
        unsigned long long* row = a.offers + (static_cast<size_t>(seg_start) + target) * a.offer_slots;
        const uint32_t s1 = offer_slot(cand, salt, a.slot_shift);
        o.where = &row[second_slot ? offer_slot_beside(s1, cand, salt) : s1];
        o.what = (static_cast<unsigned long long>(__float_as_uint(dist)) << 32) | cand;
        o.there = __hip_atomic_load(o.where, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return o;
    };
    auto send = [&](const Offer& o) {
        if (o.where && o.what < o.there) __hip_atomic_fetch_min(o.where, o.what, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    };
    // Nearest partner of a column, in registers.  A lane holds 16 rows of one column of its quadrant, in ascending row
    // order; its partner lane (the other half of the wavefront) the 16 rows in between; the other row block belongs to
    // another wavefront and is met through LDS.  Smaller distance first, then the smaller row: what a scan of the
    // column from the top finds.
    auto column_partial = [&](float best, uint32_t bi, float* part_d, uint32_t* part_i) {
        const float od = lane_xor<32>(best);
        const uint32_t oi = lane_xor<32>(bi);
        if (od < best || (od == best && oi < bi)) {
            best = od;
            bi = oi;
        }
        if (kh == 0) {
            part_d[rb * kBi + cb * 32 + t] = best;
            part_i[rb * kBi + cb * 32 + t] = bi;
        }
    };
    // ---- new x new.  The matrix is symmetric: the nearest new partner of member j is the arg-min of column j.
    // Rows and columns beyond the lists carry an infinite norm (and zero rows), so their entries come out infinite
    // without a test; the diagonal lies in the two wavefronts whose row and column blocks coincide.
    {
        const uint32_t j = cb * 32 + t;
        const float nj = L.new_norms[j];
        const bool diagonal_block = rb == cb;
        float best = FLT_MAX;
        uint32_t bi = kInvalid;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint32_t i0 = rb * 32 + 8 * q + 4 * kh;
            const float4 ni = *reinterpret_cast<const float4*>(&L.new_norms[i0]);
            const float n4[4] = {ni.x, ni.y, ni.z, ni.w};
#pragma unroll
            for (int m = 0; m < 4; m++) {
                float d = fmaxf((n4[m] + nj) - 2.f * acc_nn[4 * q + m], 0.f);
                if (diagonal_block && i0 + m == j) d = FLT_MAX;
                if (d < best) {
                    best = d;
                    bi = i0 + m;
                }
            }
        }
        column_partial(best, bi, L.part_d[0], L.part_i[0]);
    }
    if (n_old != 0) {
        // ---- new x old (rows: new, columns: old).  Columns as above (an old member's nearest new one); the rows (a new
        // member's nearest old one) run across the lanes and go through the distance tile in LDS.
        __syncthreads();   // every wave is done with the rows: the tile may overwrite them
        const uint32_t j = cb * 32 + t;
        const uint32_t col_id = j < n_old ? L.old_ids[j] : kInvalid;
        const float nj = L.old_norms[j];
        float best = FLT_MAX;
        uint32_t bi = kInvalid;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint32_t i0 = rb * 32 + 8 * q + 4 * kh;
            const float4 ni = *reinterpret_cast<const float4*>(&L.new_norms[i0]);
            const uint4 idi = *reinterpret_cast<const uint4*>(&L.new_ids[i0]);
            const float n4[4] = {ni.x, ni.y, ni.z, ni.w};
            const uint32_t id4[4] = {idi.x, idi.y, idi.z, idi.w};
#pragma unroll
            for (int m = 0; m < 4; m++) {
                float d = fmaxf((n4[m] + nj) - 2.f * acc_no[4 * q + m], 0.f);
                if (id4[m] == col_id) d = FLT_MAX;   // the same point sits in both lists: it is no partner of itself
                L.dist[i0 + m][j] = d;
                if (d < best) {
                    best = d;
                    bi = i0 + m;
                }
            }
        }
        column_partial(best, bi, L.part_d[1], L.part_i[1]);
    }
    __syncthreads();
    // ---- the offers.  Threads 2 j and 2 j + 1 own new x new column j (j < 64) or new x old column j - 64: the two row
    // blocks of a column are combined (the upper block wins ties, its rows come first), then each takes a slot.
    Offer of_column{nullptr, 0, 0}, of_row{nullptr, 0, 0};
    {
        const int which = tid >> 7;
        const uint32_t j = (tid >> 1) & 63;
        if (which == 0 || n_old != 0) {
            float best = L.part_d[which][j];
            uint32_t bi = L.part_i[which][j];
            const float od = L.part_d[which][kBi + j];
            if (od < best) {
                best = od;
                bi = L.part_i[which][kBi + j];
            }
            if (j < (which ? n_old : n_new) && bi != kInvalid)
                of_column = address((which ? L.old_ids : L.new_ids)[j], L.new_ids[bi], best, (which ? L.old_thr : L.new_thr)[j], tid & 1);
        }
    }
    if (n_old != 0) {
        // every lane of a row's four ends up with the row's nearest old member: the first two take the slots
        float best;
        uint32_t bj;
        const uint32_t me = line < n_new ? L.new_ids[line] : kInvalid;
        line_argmin<true>(L.dist, line, part, best, bj);
        if (part < 2 && line < n_new && bj != kInvalid) of_row = address(me, L.old_ids[bj], best, L.new_thr[line], part);
    }
    send(of_column);
    send(of_row);
    if (declined && a.stats) atomicAdd(&a.stats[2 * (blockIdx.x & 1023u) + 1], static_cast<unsigned long long>(declined));
}

// Six workgroups per CU (20 KB of LDS each): the join is bound by the latency of its gather -> matrix -> arg-min ->
// offer chain, so residency matters more than registers; seven would spill.  One workgroup per list.
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(6, 6))) void nnd_join_kernel(JoinArgs a, int lists) {
    extern __shared__ __align__(16) unsigned char smem[];
    if (blockIdx.x < a.num) join_list(a, *reinterpret_cast<JoinLds*>(smem), blockIdx.x, lists);
}

// The same for the rounds in which few lists are wide: a workgroup looks at the counts of a run of 16 lists (one cache
// line) and joins the wide ones among them, one after the other.  A million workgroups that look at one list each and
// leave would cost 0.4 ms a round.  Four workgroups per CU: the loop would spill at six, and the few lists there are do
// not fill them.
constexpr uint32_t kWideRun = 16;
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4))) void nnd_join_runs_kernel(JoinArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    const uint32_t first = blockIdx.x * kWideRun, mine = first + (threadIdx.x & 63u);
    const bool wide = (threadIdx.x & 63u) < kWideRun && mine < a.num && a.member_counts[static_cast<size_t>(mine) * 2] > kSamples;
    uint32_t todo = static_cast<uint32_t>(ballot(wide));   // the same in all four wavefronts
    while (todo) {
        const uint32_t j = static_cast<uint32_t>(__ffs(static_cast<int>(todo)) - 1);
        todo &= todo - 1;
        join_list(a, *reinterpret_cast<JoinLds*>(smem), first + j, kWideLists);
        __syncthreads();   // the next list overwrites what this one kept in LDS
    }
}

// ---- local join of a list with at most 32 new members (rows of up to 128 dims): one wavefront, no barrier ---------
// From the fourth round on nearly every list has fewer than 32 new members: the 64 x 64 tiles of the kernel above are
// then three quarters padding, and its four wavefronts hold registers and LDS for work one can do.  Here a wavefront
// joins one list by itself:
//  * rows go from memory straight into LDS (global_load_lds, 16 bytes a lane, 16 lanes a row: whole rows in one
//    round trip, no staging registers); the 16-byte pieces of row r are stored at slot piece ^ (r % 16), so the
//    matrix-core operand reads (lane t: row t) fall on distinct banks with rows 256 bytes apart;
//  * the operands of a block of 32 rows are then read into registers once and serve every tile the block takes part
//    in: new x new, new x old, and old x new.  The last is the transpose of the second; computing it as well (eight
//    more matrix instructions a tile) turns "a new member's nearest old one" into a column minimum like the other
//    two, taken over the 16 accumulator registers of a lane and one exchange between the halves of the wavefront, so
//    no distance ever leaves the registers;
//  * the second block of old members is fetched into the buffer of the new ones while the first tiles are computed.
constexpr uint32_t kNarrowJoinMaxDim = 128;
typedef const __attribute__((address_space(1))) void* global_ptr;
typedef __attribute__((address_space(3))) void* lds_ptr;

// Running column minimum over one 32 x 32 tile: rows row_base .. + 31 (their norms and ids in LDS), the lane's column
// with norm nj and id col_id.  A point is no partner of itself: the diagonal of new x new, and a point that sits in
// both lists.  Rows and columns beyond the lists carry an infinite norm (and zero rows) and never win.
__device__ __forceinline__ void tile_column_min(const float16v& acc, const float* row_norms, const uint32_t* row_ids, uint32_t row_base, float nj,
                                                uint32_t col_id, int kh, float& best, uint32_t& bi) {
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const uint32_t i0 = row_base + 8 * q + 4 * kh;
        const float4 ni = *reinterpret_cast<const float4*>(&row_norms[i0]);
        const uint4 idi = *reinterpret_cast<const uint4*>(&row_ids[i0]);
        const float n4[4] = {ni.x, ni.y, ni.z, ni.w};
        const uint32_t id4[4] = {idi.x, idi.y, idi.z, idi.w};
#pragma unroll
        for (int m = 0; m < 4; m++) {
            float d = fmaxf((n4[m] + nj) - 2.f * acc[4 * q + m], 0.f);
            if (id4[m] == col_id) d = FLT_MAX;
            if (d < best) {
                best = d;
                bi = i0 + m;
            }
        }
    }
}

constexpr int kWaitVm0 = 0x0F70, kWaitLgkm0 = 0xC07F;   // s_waitcnt vmcnt(0) / lgkmcnt(0), the other counters left alone

__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(3, 3))) void nnd_join_narrow_kernel(JoinArgs a, bool read_first) {
    // separate arrays, so that the compiler can tell reads of the small ones from the row buffers that fetches write
    __shared__ __attribute__((aligned(16))) _Float16 rows[32][kNarrowJoinMaxDim];   // one block of 32 members at a time
    __shared__ __attribute__((aligned(16))) uint32_t lds_new_ids[kSamples], lds_old_ids[kBi];
    __shared__ __attribute__((aligned(16))) float lds_new_norms[kSamples], lds_old_norms[kBi];
    const uint32_t node = blockIdx.x;
    const int lane = lane_id(), t = lane & 31, kh = lane >> 5;
    // ids before counts (one round trip); slots beyond a list hold what an earlier round left there
    const uint32_t got_new = a.members[static_cast<size_t>(node) * (2 * kBi) + t];
    const uint32_t got_old = a.members[static_cast<size_t>(node) * (2 * kBi) + kBi + lane];
    const uint2 mc = *reinterpret_cast<const uint2*>(a.member_counts + static_cast<size_t>(node) * 2);
    uint32_t seg_start, seg_len, state;
    locate_uniform(a.segs, node, seg_start, seg_len, &state);
    if (state == kDone) return;
    const uint32_t n_new = mc.x, n_old = mc.y;
    if (n_new == 0 || n_new > kSamples) return;   // wider lists belong to nnd_join_kernel
    const uint32_t new_id = static_cast<uint32_t>(t) < n_new ? got_new : kInvalid, old_id = static_cast<uint32_t>(lane) < n_old ? got_old : kInvalid;
    lds_new_ids[t] = new_id;
    lds_old_ids[lane] = old_id;
    __builtin_amdgcn_wave_barrier();

    // Sixteen lanes fetch one row; eight instructions fill a block of 32.  A lane whose row or piece does not exist
    // stores zeros in its place -- all such stores of a block before its first fetch, because an ordinary LDS store
    // waits for the fetches issued before it.
    const uint32_t my_row = lane >> 4, slot = lane & 15;
    auto row_ids = [&](uint32_t (&ids)[8], const uint32_t* from) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 8; i++) ids[i] = from[4 * i + my_row];
    };
    auto clear = [&](_Float16 (*buf)[kNarrowJoinMaxDim], const uint32_t (&ids)[8]) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint32_t r = 4 * i + my_row, piece = slot ^ (r & 15);
            if (ids[i] == kInvalid || piece * 8 >= a.dim_pad) *reinterpret_cast<float4*>(&buf[r][slot * 8]) = make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    auto fetch = [&](_Float16 (*buf)[kNarrowJoinMaxDim], const uint32_t (&ids)[8]) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint32_t r = 4 * i + my_row, piece = slot ^ (r & 15);
            if (ids[i] != kInvalid && piece * 8 < a.dim_pad)
                __builtin_amdgcn_global_load_lds((global_ptr)(a.half_rows + static_cast<size_t>(seg_start + ids[i]) * a.dim_pad + piece * 8), (lds_ptr)(&buf[4 * i][0]), 16, 0, 0);
        }
    };
    auto operands = [&](half8v (&X)[8], const _Float16 (*buf)[kNarrowJoinMaxDim]) {
#pragma unroll
        for (int s = 0; s < 8; s++) X[s] = *reinterpret_cast<const half8v*>(&buf[t][((2 * s + kh) ^ (t & 15)) * 8]);
    };
    const bool second_block = n_old > 32;
    uint32_t ids[8];
    row_ids(ids, lds_new_ids);
    clear(rows, ids);
    fetch(rows, ids);
    // norm and offer threshold of the lane's own members, in the same round trip
    float2 nw = make_float2(__builtin_inff(), __uint_as_float(kInvalid)), od = nw;
    if (new_id != kInvalid) nw = a.norms[seg_start + new_id];
    if (old_id != kInvalid) od = a.norms[seg_start + old_id];
    half8v A[8], B[8];
    __builtin_amdgcn_s_waitcnt(kWaitVm0);
    __builtin_amdgcn_wave_barrier();
    lds_new_norms[t] = nw.x;
    lds_old_norms[lane] = od.x;
    operands(A, rows);
    // The buffer is free once its rows are in registers: the next block sets out while tiles are computed.
    auto next_block = [&](const uint32_t* from) __attribute__((always_inline)) {
        __builtin_amdgcn_s_waitcnt(kWaitLgkm0);
        __builtin_amdgcn_wave_barrier();
        row_ids(ids, from);
        clear(rows, ids);
        fetch(rows, ids);
    };
    auto arrived = [&]() __attribute__((always_inline)) {
        __builtin_amdgcn_s_waitcnt(kWaitVm0);
        __builtin_amdgcn_wave_barrier();
        operands(B, rows);
    };
    if (n_old) next_block(lds_old_ids);
    const float x_od = lane_xor<32>(od.x);
    const uint32_t x_old = lane_xor<32>(old_id);
    const float b_norm[2] = {kh ? x_od : od.x, kh ? od.x : x_od};   // column t of old block 0 / 1, for both halves
    const uint32_t b_id[2] = {kh ? x_old : old_id, kh ? old_id : x_old};

    const uint32_t steps = (a.dim_pad + 15) / 16;
    auto tile = [&](const half8v (&X)[8], const half8v (&Y)[8]) __attribute__((always_inline)) {
        float16v acc;
#pragma unroll
        for (int r = 0; r < 16; r++) acc[r] = 0.f;
#pragma unroll
        for (int s = 0; s < 8; s++)
            if (static_cast<uint32_t>(s) < steps) acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(X[s], Y[s], acc, 0, 0, 0);
        return acc;
    };
    // the two halves of a wavefront hold alternate groups of four rows of a column: smaller distance, then smaller row
    auto settle = [&](float& best, uint32_t& bi) __attribute__((always_inline)) {
        const float other_d = lane_xor<32>(best);
        const uint32_t other_i = lane_xor<32>(bi);
        if (other_d < best || (other_d == best && other_i < bi)) {
            best = other_d;
            bi = other_i;
        }
    };
    float nn_d = FLT_MAX, on_d = FLT_MAX, no_d[2] = {FLT_MAX, FLT_MAX};
    uint32_t nn_i = kInvalid, on_i = kInvalid, no_i[2] = {kInvalid, kInvalid};
    {   // new x new: the nearest new partner of new member t
        const float16v acc = tile(A, A);
        tile_column_min(acc, lds_new_norms, lds_new_ids, 0, nw.x, new_id, kh, nn_d, nn_i);
        settle(nn_d, nn_i);
    }
    if (n_old) {
        arrived();
        if (second_block) next_block(lds_old_ids + 32);
        {   // new x old: the nearest new partner of old member t
            const float16v acc = tile(A, B);
            tile_column_min(acc, lds_new_norms, lds_new_ids, 0, b_norm[0], b_id[0], kh, no_d[0], no_i[0]);
            settle(no_d[0], no_i[0]);
        }
        {   // old x new: the nearest old partner of new member t, first block of rows
            const float16v acc = tile(B, A);
            tile_column_min(acc, lds_old_norms, lds_old_ids, 0, nw.x, new_id, kh, on_d, on_i);
        }
        if (second_block) {
            arrived();
            {
                const float16v acc = tile(A, B);
                tile_column_min(acc, lds_new_norms, lds_new_ids, 0, b_norm[1], b_id[1], kh, no_d[1], no_i[1]);
                settle(no_d[1], no_i[1]);
            }
            {
                const float16v acc = tile(B, A);
                tile_column_min(acc, lds_old_norms, lds_old_ids, 32, nw.x, new_id, kh, on_d, on_i);
            }
        }
        settle(on_d, on_i);
    }

    // ---- the offers: two atomic minima on slots of one line of the target's table; nothing comes back.  Every lane
    // has at most one offer of each kind.  The chip carries out some 27 G scattered atomic operations a second, and
    // nearly twice as many when adjacent lanes aim at one 128-byte line: so the two slots of an offer are taken by two
    // adjacent lanes in one instruction -- first the offers of the lower 32 lanes, then those of the upper 32.  And a
    // in the first rounds (read_first) a slot is read before anything is sent to it: within a round a slot only ever gets
    // smaller, so a minimum that would not get below what the read has found changes nothing and is left out.  In
    // those rounds half of them are -- copies of an offer another list has delivered, offers that lose their slot to a
    // nearer one -- and reads are an order of magnitude cheaper than atomics; later few are, and the read only adds a
    // round trip.
    const uint32_t salt = round_salt(*a.round);
    uint32_t declined = 0;
    unsigned long long* where[4];
    unsigned long long what[4], there[4];
    auto address = [&](int first, uint32_t target, uint32_t cand, float dist, uint32_t thr) __attribute__((always_inline)) {
        const bool wanted = target != kInvalid && cand != kInvalid && cand != target && cand < seg_len && dist < FLT_MAX;
        const bool stays_away = wanted && __float_as_uint(dist) >= thr;   // the target has asked offers from this distance on to stay away
        const uint64_t go = ballot(wanted && !stays_away);
        if (a.stats) declined += static_cast<uint32_t>(__popcll(ballot(stays_away)));
#pragma unroll
        for (int h = 0; h < 2; h++) {
            where[first + h] = nullptr;
            what[first + h] = 0;
            there[first + h] = 0;
            if (static_cast<uint32_t>(go >> (32 * h)) == 0u) continue;
            const int from = 32 * h + (lane >> 1);
            const uint32_t t_ = static_cast<uint32_t>(__shfl(static_cast<int>(target), from)), c_ = static_cast<uint32_t>(__shfl(static_cast<int>(cand), from));
            const uint32_t d_ = static_cast<uint32_t>(__shfl(static_cast<int>(__float_as_uint(dist)), from));
            if ((go >> from) & 1ull) {
                unsigned long long* row = a.offers + (static_cast<size_t>(seg_start) + t_) * a.offer_slots;
                const uint32_t s1 = offer_slot(c_, salt, a.slot_shift);
                where[first + h] = &row[(lane & 1) ? offer_slot_beside(s1, c_, salt) : s1];
                what[first + h] = (static_cast<unsigned long long>(d_) << 32) | c_;
                there[first + h] = read_first ? __hip_atomic_load(where[first + h], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : kNoOffer;
            }
        }
    };
    // lower half: the nearest new partner of new member t; upper half: its nearest old partner
    const uint32_t from_new = lds_new_ids[nn_i & 31u], from_old = lds_old_ids[on_i & 63u];
    const uint32_t partner = kh ? (on_i == kInvalid ? kInvalid : from_old) : (nn_i == kInvalid ? kInvalid : from_new);
    address(0, new_id, partner, kh ? on_d : nn_d, __float_as_uint(nw.y));
    // old member `lane`: its nearest new partner
    const uint32_t pick_old = kh ? no_i[1] : no_i[0];
    address(2, old_id, pick_old == kInvalid ? kInvalid : lds_new_ids[pick_old & 31u], kh ? no_d[1] : no_d[0], __float_as_uint(od.y));
#pragma unroll
    for (int i = 0; i < 4; i++)
        if (where[i] && what[i] < there[i]) __hip_atomic_fetch_min(where[i], what[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (declined && lane == 0) atomicAdd(&a.stats[2 * (blockIdx.x & 1023u) + 1], static_cast<unsigned long long>(declined));
}

// ---- merge ------------------------------------------------------------------------------------------------------
// Register bitonic network over M 64-bit keys (element e = (M/64) * lane + r), with an optional 32-bit payload.
template <int M, bool VAL>
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
                        if constexpr (VAL) { const uint32_t tv = v[r]; v[r] = v[r | J]; v[r | J] = tv; }
                    }
                }
            }
        } else {
            // Two entries with equal keys are copies of one entry (same distance, id, source and flag), so exchanging
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
                const uint64_t less = __builtin_amdgcn_ballot_w64(ok < k[r]);
                const uint64_t take = less ^ ~keep_min;
                const uint32_t lo = select_by_mask(static_cast<uint32_t>(k[r]), static_cast<uint32_t>(ok), take);
                const uint32_t hi = select_by_mask(static_cast<uint32_t>(k[r] >> 32), static_cast<uint32_t>(ok >> 32), take);
                k[r] = (static_cast<unsigned long long>(hi) << 32) | lo;
                if constexpr (VAL) v[r] = select_by_mask(v[r], lane_xor<LM>(v[r]), take);
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
__device__ __forceinline__ void bloom_bits(uint32_t id, uint32_t bloom_sets, uint32_t (&b)[3]) {
    const uint32_t base = (id % bloom_sets) * 512;
    uint32_t h = bloom_h0(id);
    b[0] = base + h % 512;
    h += bloom_h1(id);
    b[1] = base + h % 512;
    h += bloom_h1(id);
    b[2] = base + h % 512;
}

struct MergeArgs {
    uint32_t* list_ids;
    float* list_dists;
    unsigned long long* offers;  // num x SLOTS offer tables: read and emptied
    uint32_t* bloom;
    uint32_t* fwd_new;
    uint32_t* fwd_old;
    uint32_t* counts;            // num x 4
    unsigned long long* stats;   // striped: [0] offers received by the merge steps (nullable)
    Segments segs;
    uint32_t* rev_new;           // reverse lists of the next join (null: the scatter is a stage of its own)
    uint32_t* rev_old;
    uint32_t* rev_tables;
    const uint32_t* rev_thr;
    float2* norms;               // .y: the node's offer threshold
    uint32_t num, width, num_sub, bloom_sets;
};

// KNOWN_BITS: id set per wavefront (512 slots for lists of up to 192 entries + 32 offers, 1024 for the wider lists of
// degrees above 128); FILTER_WORDS: the node's Bloom filter (16 words per set of 32 entries of the internal degree).
template <uint32_t SLOTS, uint32_t KNOWN_BITS, uint32_t FILTER_WORDS>
struct MergeLds {
    unsigned long long keys[4][SLOTS];   // the node's offers, gaps closed
    unsigned long long best[4][kOfferThrRank];  // the best 32 of them (64 where a threshold is due)
    unsigned long long enter[4][kSamples];      // those that enter the list, as keys of the second sort
    uint32_t known[4][1u << KNOWN_BITS];
    uint32_t filter[4][FILTER_WORDS];
    uint32_t flags[4][kSamples];
};

// The smallest N_OUT distinct keys of keys[0 .. held), ascending, to best[0 ..); returns how many there are (at most N_OUT).
// Copies of one offer (the same pair met in several lists) are adjacent after the sort.  The network is sized by what
// the node holds.  `best` may be part of `keys`: everything is read before anything is written.
// N_OUT = 32, or 64 where the 64th is needed as well.
template <int M1, uint32_t N_OUT = kSamples>
__device__ __forceinline__ uint32_t best_offers(const unsigned long long* keys, uint32_t held, unsigned long long* best, int lane) {
    constexpr int NR = M1 / 64;
    unsigned long long k[NR];
    uint32_t none[NR];
#pragma unroll
    for (int r = 0; r < NR; r++) {
        const uint32_t e = NR * lane + r;
        k[r] = e < held ? keys[e] : kNoOffer;
    }
    Net64<M1, false>::sort(k, none, lane);
    const unsigned long long last_of_prev =
        (static_cast<unsigned long long>(static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(k[NR - 1] >> 32), 0x138, 0xf, 0xf, false))) << 32) |
        static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(k[NR - 1]), 0x138, 0xf, 0xf, false));   // wave_shr:1
    bool distinct[NR];
    uint32_t count = 0, total;
#pragma unroll
    for (int r = 0; r < NR; r++) {
        const unsigned long long prev = r == 0 ? last_of_prev : k[r - 1];
        distinct[r] = k[r] != kNoOffer && ((r == 0 && lane == 0) || prev != k[r]);
        count += distinct[r];
    }
    uint32_t rank = wave_exclusive_scan(count, total);
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int r = 0; r < NR; r++) {
        if (distinct[r]) {
            if (rank < N_OUT) best[rank] = k[r];
            rank++;
        }
    }
    __builtin_amdgcn_wave_barrier();
    return total < N_OUT ? total : N_OUT;
}

template <uint32_t SLOTS>
__device__ __forceinline__ uint32_t best_offers_sized(const unsigned long long* keys, uint32_t held, unsigned long long* best, int lane) {
    if constexpr (SLOTS > 256)
        if (held > 256) return best_offers<SLOTS>(keys, held, best, lane);
    if (held > 128) return best_offers<256>(keys, held, best, lane);
    if (held > 64) return best_offers<128>(keys, held, best, lane);
    if (held > 0) return best_offers<64>(keys, held, best, lane);
    return 0;
}

// Merge + resample, one wavefront per node.  The reference keeps, per node and round, a 32-wide sorted "device" list of
// the offers (insert_to_global_graph :509-579), merges it into the host list (update_graph :1106-1126: an id goes to
// sub-list id % num_sub, each a sorted list of 32 that rejects ids it already holds) and draws the samples of the next
// join from both (sample_graph_new :973-1001, sample_segment_graph :1073-1104).  Here:
//   old samples = the first <= 32 entries of the incoming list that are flagged old, in storage order (the reference
//                 samples them before this round's results are merged);
//   the node's offers are sorted by (distance, id) and the best 32 count; those whose id the list does not hold yet are
//   sorted together with the list, and every sub-list keeps its 32 nearest;
//   new samples = those of the best 32 that the Bloom filter has not seen; the ones entering the list are flagged old.
// M2 = size of the second network >= width + 32.
template <int M2, uint32_t SLOTS>
__global__ __launch_bounds__(256) void nnd_merge_kernel(MergeArgs a) {
    constexpr uint32_t kKnownBits = M2 > 256 ? 10 : 9;
    constexpr int kFilterPasses = M2 > 256 ? 4 : 2;   // Bloom filter words per lane: 128 words up to degree 128, 256 beyond
    __shared__ MergeLds<SLOTS, kKnownBits, 64 * kFilterPasses> L;
    constexpr int NR = M2 / 64;
    constexpr int PASSES = SLOTS / 256;
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const uint32_t node = blockIdx.x * 4 + wave;
    if (node >= a.num) return;
    const uint32_t width = a.width, num_sub = a.num_sub;
    const uint32_t bloom_words = a.bloom_sets * 16;   // at most 64 * kFilterPasses
    if (bloom_words > 64u * kFilterPasses || width + kSamples > static_cast<uint32_t>(M2)) return;   // not a launch nnd_merge makes: the filter or the list would not fit this form's LDS

    // ---- everything the node needs from memory is asked for at once: the kernel is bound by the latency of its
    // dependent memory round trips (this one, the thresholds of the sampled nodes, the slots of their reverse lists),
    // not by bandwidth or arithmetic
    unsigned long long* const table = a.offers + static_cast<size_t>(node) * SLOTS;
    uint4 t_lo[PASSES], t_hi[PASSES];
#pragma unroll
    for (int p = 0; p < PASSES; p++) {
        t_lo[p] = *reinterpret_cast<const uint4*>(table + 256 * p + 4 * lane);
        t_hi[p] = *reinterpret_cast<const uint4*>(table + 256 * p + 4 * lane + 2);
    }
    uint32_t l_id[NR];
    float l_dist[NR];
#pragma unroll
    for (int r = 0; r < NR; r++) {
        const uint32_t e = NR * lane + r;
        l_id[r] = e < width ? a.list_ids[static_cast<size_t>(node) * width + e] : kInvalid;
        l_dist[r] = e < width ? a.list_dists[static_cast<size_t>(node) * width + e] : FLT_MAX;
    }
    uint32_t bloom_in[kFilterPasses];
#pragma unroll
    for (int j = 0; j < kFilterPasses; j++) bloom_in[j] = lane + 64u * j < bloom_words ? a.bloom[static_cast<size_t>(node) * bloom_words + lane + 64 * j] : 0u;
    const uint32_t in_force = __float_as_uint(a.norms[node].y);
    uint32_t seg_start, seg_len, state;
    const uint32_t seg = locate_uniform(a.segs, node, seg_start, seg_len, &state);
    if (state == kDone) return;

    unsigned long long* keys = L.keys[wave];
    unsigned long long* best = L.best[wave];
    unsigned long long* enter = L.enter[wave];
    uint32_t* known = L.known[wave];
    uint32_t* filter = L.filter[wave];
    uint32_t* flags = L.flags[wave];
    for (uint32_t i = lane; i < (1u << kKnownBits); i += 64) known[i] = kInvalid;
#pragma unroll
    for (int j = 0; j < kFilterPasses; j++)
        if (lane + 64u * j < bloom_words) filter[lane + 64 * j] = bloom_in[j];
    __builtin_amdgcn_wave_barrier();

    // ---- the incoming list, in storage order; its ids go into the wavefront's id set
    unsigned long long k[NR];
    uint32_t v[NR];
    uint32_t old_count = 0;
#pragma unroll
    for (int r = 0; r < NR; r++) {
        k[r] = ~0ull;
        v[r] = 0;
        const uint32_t id = l_id[r];
        if (id != kInvalid) {
            k[r] = (static_cast<unsigned long long>(__float_as_uint(l_dist[r])) << 32) | (static_cast<unsigned long long>(id & ~kOld) << 1);
            v[r] = id & kOld;
            old_count += (id & kOld) != 0;
            hash_insert(known, kKnownBits, id & ~kOld);
        }
    }
    // old samples from the incoming list (element order = storage order = the reference's scan order).  With the
    // scatter fused in, a sample also enters the reverse list of the node it names: first the threshold that node has
    // announced is asked for, further down a slot, and the entry is stored at the very end.
    const uint32_t me = node - seg_start;
    uint32_t total_old;
    size_t old_target[NR];
    uint32_t old_thr[NR], old_pos[NR];
    {
        uint32_t rank = wave_exclusive_scan(old_count, total_old);
#pragma unroll
        for (int r = 0; r < NR; r++) {
            old_target[r] = ~static_cast<size_t>(0);
            old_thr[r] = 0;
            if (k[r] != ~0ull && (v[r] & kOld)) {
                if (rank < kSamples) {
                    const uint32_t id = static_cast<uint32_t>((k[r] >> 1) & 0x7fffffffull);
                    a.fwd_old[static_cast<size_t>(node) * kSamples + rank] = id;
                    if (a.rev_old) {
                        old_target[r] = static_cast<size_t>(seg_start) + id;
                        old_thr[r] = a.rev_thr[old_target[r] * 2 + 1];
                    }
                }
                rank++;
            }
        }
    }

    // ---- this round's offers: the node's table, four slots per lane and pass, emptied where something was found
    uint32_t held;
    {
        unsigned long long o[PASSES][4];
        uint32_t mine = 0;
#pragma unroll
        for (int p = 0; p < PASSES; p++) {
            o[p][0] = (static_cast<unsigned long long>(t_lo[p].y) << 32) | t_lo[p].x;
            o[p][1] = (static_cast<unsigned long long>(t_lo[p].w) << 32) | t_lo[p].z;
            o[p][2] = (static_cast<unsigned long long>(t_hi[p].y) << 32) | t_hi[p].x;
            o[p][3] = (static_cast<unsigned long long>(t_hi[p].w) << 32) | t_hi[p].z;
            if ((o[p][0] & o[p][1] & o[p][2] & o[p][3]) != kNoOffer) {
                const uint4 empty = make_uint4(kInvalid, kInvalid, kInvalid, kInvalid);
                *reinterpret_cast<uint4*>(table + 256 * p + 4 * lane) = empty;
                *reinterpret_cast<uint4*>(table + 256 * p + 4 * lane + 2) = empty;
            }
#pragma unroll
            for (int j = 0; j < 4; j++) mine += o[p][j] != kNoOffer;
        }
        uint32_t at = wave_exclusive_scan(mine, held);
#pragma unroll
        for (int p = 0; p < PASSES; p++)
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (o[p][j] != kNoOffer) keys[at++] = o[p][j];
    }
    __builtin_amdgcn_wave_barrier();
    uint32_t n_best;
    uint32_t next_thr;
    if (held < SLOTS / 8 * kOfferCrowdedEighths) {
        n_best = best_offers_sized<SLOTS>(keys, held, best, lane);
        // a threshold that is in force stays while the node still receives plenty of offers and its best 32 are complete
        next_thr = held >= kOfferKeepHeld && n_best == kSamples ? in_force : kInvalid;
    } else {
        // A crowded table: thousands of offers may have met here, and most of the round's cost for this node was their
        // atomics on these few lines.  The distance of the 64th best offer becomes the node's threshold for the next join.
        const uint32_t n64 = held > 256 ? best_offers<SLOTS, kOfferThrRank>(keys, held, best, lane) : best_offers<256, kOfferThrRank>(keys, held, best, lane);
        n_best = n64 < kSamples ? n64 : kSamples;
        next_thr = n64 == kOfferThrRank ? static_cast<uint32_t>(best[kOfferThrRank - 1] >> 32) : kInvalid;
    }
    if (lane == 0 && next_thr != in_force) a.norms[node].y = __uint_as_float(next_thr);

    // ---- the best 32 offers, one per lane: new samples, and which of them enter the list
    uint32_t total_new = 0;
    size_t new_target = ~static_cast<size_t>(0);
    uint32_t new_thr = 0, new_pos = 0;
    {
        const bool mine = static_cast<uint32_t>(lane) < n_best;
        const unsigned long long key = mine ? best[lane] : kNoOffer;
        const uint32_t id = static_cast<uint32_t>(key);
        const bool take = mine && id < seg_len;
        bool fresh = false;
        uint32_t b[3];
        if (take) {
            bloom_bits(id, a.bloom_sets, b);
            fresh = ((filter[b[0] >> 5] >> (b[0] & 31)) & (filter[b[1] >> 5] >> (b[1] & 31)) & (filter[b[2] >> 5] >> (b[2] & 31)) & 1u) == 0;
        }
        // an id the list holds (whatever its distance there) is rejected, as insert_to_ordered_list :916-943 does
        const bool enters = take && hash_insert(known, kKnownBits, id) != 0;
        const uint64_t fm = ballot(fresh);
        total_new = __popcll(fm);
        __builtin_amdgcn_wave_barrier();   // every lane has tested the filter before bits are added
        if (fresh) {   // at most 32 of them: all become samples
            a.fwd_new[static_cast<size_t>(node) * kSamples + prefix_count(fm)] = id;
            if (a.rev_new) {
                new_target = static_cast<size_t>(seg_start) + id;
                new_thr = a.rev_thr[new_target * 2];
            }
            atomicOr(&filter[b[0] >> 5], 1u << (b[0] & 31));
            atomicOr(&filter[b[1] >> 5], 1u << (b[1] & 31));
            atomicOr(&filter[b[2] >> 5], 1u << (b[2] & 31));
        }
        const unsigned long long entering = ((key >> 32) << 32) | (static_cast<unsigned long long>(id) << 1) | 1ull;
        if constexpr (NR == 1) {
            // One sub-list: the list is in ascending order from the second round on, and so are the offers.  The
            // entering ones are packed in descending order behind it, which makes the whole a bitonic sequence that
            // six exchange steps sort.
            const uint64_t em = ballot(enters);
            if (lane < static_cast<int>(kSamples)) enter[lane] = ~0ull;
            __builtin_amdgcn_wave_barrier();
            if (enters) {
                const uint32_t at = kSamples - 1 - prefix_count(em);
                enter[at] = entering;
                flags[at] = fresh ? kOld : 0u;
            }
        } else if (lane < static_cast<int>(kSamples)) {
            enter[lane] = enters ? entering : ~0ull;
            flags[lane] = fresh ? kOld : 0u;
        }
    }
    // the slots of the reverse entries (add_rev_edges_kernel :490-507 for one sample each): a sample whose source is
    // not below the threshold of the node it names stays away
#pragma unroll
    for (int r = 0; r < NR; r++) {
        if (old_target[r] != ~static_cast<size_t>(0) && me >= old_thr[r]) old_target[r] = ~static_cast<size_t>(0);
        old_pos[r] = old_target[r] != ~static_cast<size_t>(0) ? atomicAdd(&a.counts[old_target[r] * 4 + 3], 1u) : 0u;
    }
    if (new_target != ~static_cast<size_t>(0) && me >= new_thr) new_target = ~static_cast<size_t>(0);
    if (new_target != ~static_cast<size_t>(0)) new_pos = atomicAdd(&a.counts[new_target * 4 + 2], 1u);

    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int r = 0; r < NR; r++) {
        const uint32_t e = NR * lane + r;
        if (e >= width && e < width + kSamples) {
            k[r] = enter[e - width];
            v[r] = flags[e - width];
        }
    }
    if constexpr (NR == 1) {
        const unsigned long long before =
            (static_cast<unsigned long long>(static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(k[0] >> 32), 0x138, 0xf, 0xf, false))) << 32) |
            static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(k[0]), 0x138, 0xf, 0xf, false));   // wave_shr:1
        const bool out_of_order = lane > 0 && lane < static_cast<int>(kSamples) && before > k[0];
        if (ballot(out_of_order) == 0)
            Net64<M2, true>::template merge_from<M2, M2 / 2>(k, v, lane);
        else   // the random start lists, or a list a caller has replaced
            Net64<M2, true>::sort(k, v, lane);
    } else {
        Net64<M2, true>::sort(k, v, lane);
    }

    // ---- every sub-list keeps its 32 nearest: rank of an entry among those of its sub-list, in sorted order
    const unsigned long long last_of_prev =
        (static_cast<unsigned long long>(static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(k[NR - 1] >> 32), 0x138, 0xf, 0xf, false))) << 32) |
        static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(k[NR - 1]), 0x138, 0xf, 0xf, false));   // wave_shr:1
    bool valid[NR];
    uint32_t sub[NR], slot[NR];
#pragma unroll
    for (int r = 0; r < NR; r++) {
        const unsigned long long prev = r == 0 ? last_of_prev : k[r - 1];
        const bool head = (r == 0 && lane == 0);
        // a repeated entry (the random start lists of a very small partition) is dropped
        valid[r] = k[r] != ~0ull && (head || (prev >> 1) != (k[r] >> 1));
        const uint32_t id = static_cast<uint32_t>((k[r] >> 1) & 0x7fffffffull);
        sub[r] = num_sub == 1 ? 0u : id % num_sub;
        slot[r] = kInvalid;
    }
    for (uint32_t s = 0; s < num_sub; s++) {
        uint32_t count = 0, total;
#pragma unroll
        for (int r = 0; r < NR; r++) count += valid[r] && sub[r] == s;
        uint32_t rank = wave_exclusive_scan(count, total);
#pragma unroll
        for (int r = 0; r < NR; r++) {
            if (valid[r] && sub[r] == s) {
                if (rank < kSamples) slot[r] = rank * num_sub + s;
                rank++;
            }
        }
        for (uint32_t j = total + lane; j < kSamples; j += 64) {   // the unfilled tail of this sub-list
            a.list_ids[static_cast<size_t>(node) * width + j * num_sub + s] = kInvalid;
            a.list_dists[static_cast<size_t>(node) * width + j * num_sub + s] = FLT_MAX;
        }
    }
    uint32_t inserted = 0;
#pragma unroll
    for (int r = 0; r < NR; r++) {
        if (slot[r] != kInvalid) {
            const uint32_t id = static_cast<uint32_t>((k[r] >> 1) & 0x7fffffffull);
            a.list_ids[static_cast<size_t>(node) * width + slot[r]] = id | v[r];
            a.list_dists[static_cast<size_t>(node) * width + slot[r]] = __uint_as_float(static_cast<uint32_t>(k[r] >> 32));
            inserted += static_cast<uint32_t>(k[r] & 1ull);
        }
    }
    // update_counter (update_graph :1106-1126): insertions on every 100th row, per partition
    if (node % kCounterInterval == 0) {
        uint32_t total_inserted;
        wave_exclusive_scan(inserted, total_inserted);
        if (lane == 0 && total_inserted) atomicAdd(&a.segs.updates[seg], total_inserted);
    }
    __builtin_amdgcn_wave_barrier();
    for (uint32_t w = lane; w < bloom_words; w += 64) a.bloom[static_cast<size_t>(node) * bloom_words + w] = filter[w];
    if (lane == 0) {
        a.counts[static_cast<size_t>(node) * 4 + 0] = total_new;
        a.counts[static_cast<size_t>(node) * 4 + 1] = total_old < kSamples ? total_old : kSamples;
        if (!a.rev_new) {   // with the scatter fused in, other wavefronts are adding to these two right now; the join clears them
            a.counts[static_cast<size_t>(node) * 4 + 2] = 0;
            a.counts[static_cast<size_t>(node) * 4 + 3] = 0;
        }
        // striped over 1024 slots: one shared address would serialise every wavefront of the launch
        if (a.stats && held) atomicAdd(&a.stats[2 * (blockIdx.x & 1023u)], static_cast<unsigned long long>(held));
    }
    // ---- the reverse entries, now that their slots have come back: into the list, or past its end into the overflow table
#pragma unroll
    for (int r = 0; r < NR; r++) {
        if (old_target[r] != ~static_cast<size_t>(0)) {
            if (old_pos[r] < kRevCap)
                a.rev_old[old_target[r] * kRevStride + old_pos[r]] = me;
            else
                reverse_insert(a.rev_tables + (old_target[r] * 2 + 1) * kRevSlots, me);
        }
    }
    if (new_target != ~static_cast<size_t>(0)) {
        if (new_pos < kRevCap)
            a.rev_new[new_target * kRevStride + new_pos] = me;
        else
            reverse_insert(a.rev_tables + new_target * 2 * kRevSlots, me);
    }
}

// Termination test of GNND::build's update_and_sample (nn_descent.cuh:1270-1284): a partition whose sampled update
// count falls below termination_threshold * rows * dim / 100 (rows = all rows of the build, as in the reference) runs
// one more round -- the reference has already started that round's join when the host notices -- and then rests.
__global__ void nnd_converge_kernel(Segments segs, float limit, uint32_t* round) {
    const uint32_t s = blockIdx.x * blockDim.x + threadIdx.x;
    if (s == 0) round[0] += 1;
    if (s >= segs.count) return;
    const uint32_t state = segs.state[s];
    if (state == kLastRound) {
        segs.state[s] = kDone;
    } else if (state == kActive && static_cast<float>(segs.updates[s]) < limit) {
        segs.state[s] = kLastRound;
    }
    segs.updates[s] = 0;
}

// ---- finalize (shrink step :1376-1402): the `degree` nearest entries of each list; unfilled slots get a pseudo-random id.
// The reference copies whole sub-lists in storage order (and so never returns an id of the last sub-list when the
// degree is above 32); here the sub-lists are merged by (distance, id) first.
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

template <int M>
__global__ __launch_bounds__(256) void nnd_finalize_kernel(const uint32_t* list_ids, const float* list_dists, uint32_t num, uint32_t width,
                                                           uint32_t degree, Segments segs, uint32_t* knn_graph) {
    constexpr int NR = M / 64;
    const int lane = lane_id();
    const uint32_t node = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (node >= num) return;
    uint32_t start, len;
    locate_uniform(segs, node, start, len);
    unsigned long long k[NR];
    uint32_t none[NR];
    uint32_t count = 0, total;
#pragma unroll
    for (int r = 0; r < NR; r++) {
        const uint32_t e = NR * lane + r;
        k[r] = ~0ull;
        if (e < width) {
            const uint32_t entry = list_ids[static_cast<size_t>(node) * width + e];
            const uint32_t id = entry & ~kOld;
            if (entry != kInvalid && id < len) {
                k[r] = (static_cast<unsigned long long>(__float_as_uint(list_dists[static_cast<size_t>(node) * width + e])) << 32) | id;
                count++;
            }
        }
    }
    wave_exclusive_scan(count, total);
    Net64<M, false>::sort(k, none, lane);
#pragma unroll
    for (int r = 0; r < NR; r++) {
        const uint32_t e = NR * lane + r;
        if (e < degree) knn_graph[static_cast<size_t>(node) * degree + e] = e < total ? static_cast<uint32_t>(k[r]) : xorshift32(node * width + e) % (len ? len : 1);
    }
}

}  // namespace glide

using namespace glide;

namespace {
uint32_t nnd_width(uint32_t degree) { return round_up32(static_cast<uint32_t>(degree * (degree <= 32 ? 1.0 : 1.3))); }  // nn_descent.cuh:1427-1428
size_t align256(size_t x) { return (x + 255) / 256 * 256; }
constexpr uint32_t kMaxWidth = 480;   // width + 32 offers fit one 512-key network; degree 256, the widest the build searches take, needs 352

struct NndLayout {
    size_t half_rows, norms, list_ids, list_dists, fwd_new, fwd_old, rev_new, rev_old, rev_tables, rev_thr, counts, members, member_counts, offers, bloom, stats,
        seg_state, seg_updates, round, total;
    uint32_t width, dim_pad, bloom_sets;
};
NndLayout nnd_layout(uint32_t num, uint32_t dim, uint32_t degree) {
    NndLayout l;
    l.width = nnd_width(degree);
    l.dim_pad = (dim + 7) / 8 * 8;
    l.bloom_sets = nnd_width(static_cast<uint32_t>(1.5 * degree)) / 32;   // internal degree / 32 (nn_descent.cuh:962, params.cuh:23-24)
    const size_t n = num;
    size_t off = 0;
    auto take = [&off](size_t bytes) { size_t o = off; off += align256(bytes); return o; };
    l.half_rows = take(n * l.dim_pad * 2);
    l.norms = take(n * 8);
    l.list_ids = take(n * l.width * 4);
    l.list_dists = take(n * l.width * 4);
    l.fwd_new = take(n * kSamples * 4);
    l.fwd_old = take(n * kSamples * 4);
    l.rev_new = take(n * kRevStride * 4);
    l.rev_old = take(n * kRevStride * 4);
    // the next two are adjacent: one fill empties the overflow tables of the reverse samples and withdraws their thresholds
    l.rev_tables = take(n * 2 * kRevSlots * 4);
    l.rev_thr = take(n * 8);
    l.counts = take(n * 16);
    l.members = take(n * 2 * kBi * 4);
    l.member_counts = take(n * 8);
    l.offers = take(n * offer_slots_for(l.width) * 8);
    l.bloom = take(n * l.bloom_sets * 64);
    l.stats = take(1024 * 16);
    l.seg_state = take(kMaxSegments * 4);
    l.seg_updates = take(kMaxSegments * 4);
    l.round = take(4);
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
    float2* norms;
    uint32_t* list_ids;
    float* list_dists;
    uint32_t *fwd_new, *fwd_old, *rev_new, *rev_old, *rev_tables, *rev_thr, *counts, *members, *member_counts, *round;
    unsigned long long* offers;
    uint32_t* bloom;
    unsigned long long* stats;
    Segments segs;
    uint32_t n;
    hipStream_t s;
};

bool nnd_degree_supported(uint32_t knn_degree) {
    return knn_degree <= 256 && nnd_width(knn_degree) <= kMaxWidth && nnd_width(static_cast<uint32_t>(1.5 * knn_degree)) / 32 <= 16;   // Bloom filter within 256 words
}

int nnd_context(NndCtx& c, uint32_t reorder_num, uint32_t dim, const uint32_t* segment_starts, const uint32_t* segment_lengths,
                uint32_t segment_num, uint32_t knn_degree, void* workspace, size_t workspace_bytes, void* stream) {
    if (!segment_starts || !segment_lengths || !workspace) return GLIDE_ERR_BAD_ARGUMENT;
    if (dim == 0 || segment_num == 0 || knn_degree == 0 || reorder_num == 0) return GLIDE_ERR_BAD_ARGUMENT;
    if (segment_num > kMaxSegments) return GLIDE_ERR_UNSUPPORTED;
    if (!nnd_degree_supported(knn_degree) || dim % 4 != 0) return GLIDE_ERR_UNSUPPORTED;
    // one thread per list slot / per sample: the products must fit the 32-bit launch arithmetic
    if (static_cast<unsigned long long>(reorder_num) * nnd_width(knn_degree) >= 0xffffffffull || reorder_num >= (1u << 26)) return GLIDE_ERR_UNSUPPORTED;
    c.l = nnd_layout(reorder_num, dim, knn_degree);
    if (workspace_bytes < c.l.total || reinterpret_cast<uintptr_t>(workspace) % 16) return GLIDE_ERR_BAD_ARGUMENT;
    unsigned char* w = static_cast<unsigned char*>(workspace);
    c.half_rows = reinterpret_cast<_Float16*>(w + c.l.half_rows);
    c.norms = reinterpret_cast<float2*>(w + c.l.norms);
    c.list_ids = reinterpret_cast<uint32_t*>(w + c.l.list_ids);
    c.list_dists = reinterpret_cast<float*>(w + c.l.list_dists);
    c.fwd_new = reinterpret_cast<uint32_t*>(w + c.l.fwd_new);
    c.fwd_old = reinterpret_cast<uint32_t*>(w + c.l.fwd_old);
    c.rev_new = reinterpret_cast<uint32_t*>(w + c.l.rev_new);
    c.rev_old = reinterpret_cast<uint32_t*>(w + c.l.rev_old);
    c.rev_tables = reinterpret_cast<uint32_t*>(w + c.l.rev_tables);
    c.rev_thr = reinterpret_cast<uint32_t*>(w + c.l.rev_thr);
    c.counts = reinterpret_cast<uint32_t*>(w + c.l.counts);
    c.members = reinterpret_cast<uint32_t*>(w + c.l.members);
    c.member_counts = reinterpret_cast<uint32_t*>(w + c.l.member_counts);
    c.offers = reinterpret_cast<unsigned long long*>(w + c.l.offers);
    c.bloom = reinterpret_cast<uint32_t*>(w + c.l.bloom);
    c.stats = reinterpret_cast<unsigned long long*>(w + c.l.stats);
    c.round = reinterpret_cast<uint32_t*>(w + c.l.round);
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
    rc = glide_hip_fill_u32(c.segs.state, 0u, 2 * kMaxSegments + 1, c.s);   // state, updates and the round count are adjacent
    if (rc != GLIDE_OK) return rc;
    // empty overflow tables (their bounds included: nothing turned away yet), empty offer tables
    rc = glide_hip_fill_u32(c.rev_tables, kInvalid, (c.l.counts - c.l.rev_tables) / 4, c.s);
    if (rc != GLIDE_OK) return rc;
    rc = glide_hip_fill_u32(reinterpret_cast<uint32_t*>(c.offers), kInvalid, static_cast<size_t>(c.n) * offer_slots_for(c.l.width) * 2, c.s);
    if (rc != GLIDE_OK) return rc;
    hipLaunchKernelGGL(nnd_prepare_kernel, dim3(ceil_div(c.n, 4)), dim3(256), 0, c.s, data, c.n, dim, c.l.dim_pad, c.half_rows, c.norms);
    hipLaunchKernelGGL(nnd_init_kernel, dim3(ceil_div(c.n * c.l.width, 256)), dim3(256), 0, c.s, c.list_ids, c.list_dists, c.n, c.l.width, c.segs, seed);
    // first samples come from the random lists (sample_graph(true), nn_descent.cuh:1266); later ones from the merge
    hipLaunchKernelGGL(nnd_sample_kernel, dim3(ceil_div(c.n, 4)), dim3(256), 0, c.s, c.list_ids, c.n, c.l.width, c.segs, c.fwd_new, c.fwd_old, c.counts);
    return launch_status();
}

int nnd_reverse(const NndCtx& c) {
    hipLaunchKernelGGL(nnd_reverse_kernel, dim3(ceil_div(c.n, 4)), dim3(256), 0, c.s, c.fwd_new, c.fwd_old, c.counts, c.rev_new, c.rev_old,
                       c.rev_tables, c.rev_thr, c.n, c.segs);
    return launch_status();
}

// few_wide: most lists are expected to have at most 32 new members (the rule once the first rounds are over)
// early: one of the first rounds, in which many offers are copies of one another
int nnd_join(const NndCtx& c, bool with_stats, bool few_wide = false, bool early = true) {
    GLIDE_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(&nnd_join_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      static_cast<int>(sizeof(JoinLds))));
    GLIDE_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(&nnd_join_runs_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      static_cast<int>(sizeof(JoinLds))));
    JoinArgs ja{c.half_rows, c.norms, c.fwd_new, c.fwd_old, c.rev_new, c.rev_old, c.rev_tables, c.rev_thr, c.counts, c.members, c.member_counts, c.offers, offer_slots_for(c.l.width),
                offer_slots_for(c.l.width) == 512 ? 23u : 24u, c.round, with_stats ? c.stats : nullptr, c.n, c.l.dim_pad, c.segs};
    hipLaunchKernelGGL(nnd_members_kernel, dim3(ceil_div(c.n, 4)), dim3(256), 0, c.s, ja);
    // lists with at most 32 new members go to the one-wavefront kernel, the others to the workgroup kernel; each passes
    // over the other's lists
    const bool narrow = c.l.dim_pad <= kNarrowJoinMaxDim;
    if (narrow && few_wide)
        hipLaunchKernelGGL(nnd_join_runs_kernel, dim3(ceil_div(c.n, kWideRun)), dim3(256), sizeof(JoinLds), c.s, ja);
    else
        hipLaunchKernelGGL(nnd_join_kernel, dim3(c.n), dim3(256), sizeof(JoinLds), c.s, ja, narrow ? kWideLists : kAllLists);
    if (narrow) hipLaunchKernelGGL(nnd_join_narrow_kernel, dim3(c.n), dim3(64), 0, c.s, ja, early);
    return launch_status();
}

// scatter_reverse: the new and old samples a node draws enter the reverse tables of their targets right away
// (what the next round's nnd_reverse would do), while the sort of other nodes keeps the vector ALU busy
int nnd_merge(const NndCtx& c, bool with_stats, bool scatter_reverse = false) {
    MergeArgs ma{c.list_ids, c.list_dists, c.offers, c.bloom, c.fwd_new, c.fwd_old, c.counts, with_stats ? c.stats : nullptr, c.segs,
                 scatter_reverse ? c.rev_new : nullptr, scatter_reverse ? c.rev_old : nullptr, scatter_reverse ? c.rev_tables : nullptr, c.rev_thr, c.norms,
                 c.n, c.l.width, c.l.width / kSamples, c.l.bloom_sets};
    // The kernel is chosen by the keys of its second sort (list + 32 offers) and by the node's Bloom filter, which the
    // forms up to 256 keys hold in 128 words of LDS: degrees 129 .. 170 have lists of 224 entries but filters of 160 words.
    const uint32_t m = c.l.width + kSamples;
    const bool small_filter = c.l.bloom_sets * 16 <= 128;
    if (c.l.bloom_sets * 16 > 256 || m > 512) return GLIDE_ERR_UNSUPPORTED;   // nnd_degree_supported keeps such degrees out
    if (m <= 64 && small_filter)
        hipLaunchKernelGGL((nnd_merge_kernel<64, kOfferSlotsNarrow>), dim3(ceil_div(c.n, 4)), dim3(256), 0, c.s, ma);
    else if (m <= 128 && small_filter)
        hipLaunchKernelGGL((nnd_merge_kernel<128, kOfferSlotsWide>), dim3(ceil_div(c.n, 4)), dim3(256), 0, c.s, ma);
    else if (m <= 256 && small_filter)
        hipLaunchKernelGGL((nnd_merge_kernel<256, kOfferSlotsWide>), dim3(ceil_div(c.n, 4)), dim3(256), 0, c.s, ma);
    else
        hipLaunchKernelGGL((nnd_merge_kernel<512, kOfferSlotsWide>), dim3(ceil_div(c.n, 4)), dim3(256), 0, c.s, ma);
    return launch_status();
}

int nnd_converge(const NndCtx& c, uint32_t dim, float termination_threshold) {
    // update_counter < termination_threshold * nrow * dim / counter_interval (nn_descent.cuh:1280), evaluated in float
    const float limit = termination_threshold * static_cast<float>(c.n) * static_cast<float>(dim) / static_cast<float>(kCounterInterval);
    hipLaunchKernelGGL(nnd_converge_kernel, dim3(ceil_div(c.segs.count, 256)), dim3(256), 0, c.s, c.segs, limit, c.round);
    return launch_status();
}

int nnd_finalize(const NndCtx& c, uint32_t knn_degree, uint32_t* knn_graph, unsigned long long* stats_out) {
    if (c.l.width <= 64)
        hipLaunchKernelGGL(nnd_finalize_kernel<64>, dim3(ceil_div(c.n, 4)), dim3(256), 0, c.s, c.list_ids, c.list_dists, c.n, c.l.width, knn_degree, c.segs, knn_graph);
    else if (c.l.width <= 128)
        hipLaunchKernelGGL(nnd_finalize_kernel<128>, dim3(ceil_div(c.n, 4)), dim3(256), 0, c.s, c.list_ids, c.list_dists, c.n, c.l.width, knn_degree, c.segs, knn_graph);
    else if (c.l.width <= 256)
        hipLaunchKernelGGL(nnd_finalize_kernel<256>, dim3(ceil_div(c.n, 4)), dim3(256), 0, c.s, c.list_ids, c.list_dists, c.n, c.l.width, knn_degree, c.segs, knn_graph);
    else
        hipLaunchKernelGGL(nnd_finalize_kernel<512>, dim3(ceil_div(c.n, 4)), dim3(256), 0, c.s, c.list_ids, c.list_dists, c.n, c.l.width, knn_degree, c.segs, knn_graph);
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
        if ((rc = nnd_join(c, stats_out != nullptr, it >= 3, it < 4)) != GLIDE_OK) return rc;
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
    if (!nnd_degree_supported(knn_degree) || dim % 4 != 0) return GLIDE_ERR_UNSUPPORTED;
    const NndLayout l = nnd_layout(reorder_num, dim, knn_degree);
    out->half_rows = l.half_rows; out->norms = l.norms; out->list_ids = l.list_ids; out->list_dists = l.list_dists;
    out->fwd_new = l.fwd_new; out->fwd_old = l.fwd_old; out->rev_new = l.rev_new; out->rev_old = l.rev_old; out->rev_tables = l.rev_tables; out->rev_thr = l.rev_thr;
    out->counts = l.counts; out->members = l.members; out->member_counts = l.member_counts; out->offers = l.offers; out->bloom = l.bloom;
    out->segment_state = l.seg_state; out->segment_updates = l.seg_updates; out->round = l.round; out->total = l.total;
    out->width = l.width; out->reverse_cap = kRevCap; out->reverse_stride = kRevStride; out->offer_slots = offer_slots_for(l.width); out->reverse_slots = kRevSlots; out->row_halfs = l.dim_pad; out->bloom_sets = l.bloom_sets; out->reserved = 0;
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

int glide_hip_nnd_sample(uint32_t reorder_num, uint32_t dim, const uint32_t* segment_starts, const uint32_t* segment_lengths,
                         uint32_t segment_num, uint32_t knn_degree, void* workspace, size_t workspace_bytes, void* stream) {
    NndCtx c;
    int rc = nnd_context(c, reorder_num, dim, segment_starts, segment_lengths, segment_num, knn_degree, workspace, workspace_bytes, stream);
    if (rc != GLIDE_OK) return rc;
    hipLaunchKernelGGL(nnd_sample_kernel, dim3(ceil_div(c.n, 4)), dim3(256), 0, c.s, c.list_ids, c.n, c.l.width, c.segs, c.fwd_new, c.fwd_old, c.counts);
    return launch_status();
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
    return rc != GLIDE_OK ? rc : nnd_join(c, true);
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
