// Beam-search core for one item per 64-lane wavefront (search, sub-graph build, refine all use it).
//
// Reference semantics: search_kernel.cuh:433-482 / graph_kernel.cuh:16-63 (one iteration), :9-37 and :97-148
// (candidate sort, beam merge), :292-325 (parent selection), :327-334 (hash restore), :336-391 (expansion).
//
// Layout: the beam (MAX_BEAM entries) lives in registers, element e = NB*lane + r, ascending, explored flag in
// the id's MSB.  The D candidates of one expansion are produced into LDS by graph-row slot, pulled into
// registers with the reference's strided->blocked permutation, sorted by the wave network and staged back to
// LDS so that beam element e can pick candidate MAX_BEAM-1-e (the half-cleaner).  The visited set is an LDS
// open-addressing table.  Data rows are gathered several at a time (one lane group each, 16 B per lane and load).
#pragma once
#include "bitonic.hpp"

namespace glide {

struct BeamParams {
    uint32_t beam, degree, dim, hash_bit, reset_interval, max_iterations, min_iterations;
    int metric;
};

constexpr uint32_t kCounterStripes = 256;

struct BeamCounters {  // wave-uniform tallies for traffic accounting
    uint32_t iterations = 0, rows_scored = 0, graph_rows = 0;
};

template <int MAX_CAND>
struct BeamLds {  // per-wave LDS (the hash table follows, 1 << hash_bit words)
    uint32_t cand_id[MAX_CAND];
    float cand_dist[MAX_CAND];
    uint32_t vlist[MAX_CAND];
};

// Beams the kernels take: up to 512 (the reference's widest bucket, kernel_config.cuh:41-48); above 256 a multiple of 16, so
// that each half of the beam is whole lanes of eight entries (the reference's adjust_search_params, params.cuh:82-99, only
// ever hands out multiples of 32).
inline bool beam_supported(uint32_t beam) { return beam <= 512 && (beam <= 256 || beam % 16 == 0); }

// Host-side size of the candidate lists for a degree bucket (the hash table follows them in the dynamic LDS).
inline size_t beam_lds_bytes(uint32_t degree) {
    return degree <= 64 ? sizeof(BeamLds<64>) : degree <= 128 ? sizeof(BeamLds<128>) : sizeof(BeamLds<256>);
}

__device__ __forceinline__ void wave_sync() { __syncthreads(); }  // workgroup == one wavefront
// The same point in a wavefront that shares its workgroup with others (TEAM): a workgroup barrier would wait for them.
// LDS instructions of one wavefront execute in program order; what is needed between a store and a dependent load of
// another lane is that the compiler keeps that order, which a wavefront-scope fence does.
template <bool TEAM>
__device__ __forceinline__ void wave_sync_in() {
    if constexpr (TEAM) {
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
    } else {
        __syncthreads();
    }
}

// Where score_list reads the reference row from: registers (one copy per wavefront) ...
template <int DIMV>
struct RefInRegs {
    const RowRegs<DIMV>& r;
    __device__ __forceinline__ float4 chunk(int c, int) const { return r.v[c]; }
};
// ... or LDS, laid out as the loads of one lane group would hold it (chunk c of lane t at [c * LPR + t]): the wavefronts
// of a team share one copy and keep their registers for rows in flight.  The two lane groups of a wide row read the same
// addresses (a broadcast), adjacent lanes adjacent 16-byte words: no bank conflicts.
template <int DIMV>
struct RefInLds {
    const float4* q;
    __device__ __forceinline__ float4 chunk(int c, int t) const { return q[c * RowShape<DIMV>::LPR + t]; }
};

// Distances from a reference row to `count` listed rows, RowShape<DIMV>::ROWS rows per step (one per lane group), U steps
// in flight.  id_of(idx) -> row id of list entry idx; out(idx, dist) is called by one lane per scored row.  A team of
// `members` wavefronts splits the list in runs of ROWS * U entries, member `member` taking every members-th run; the sum
// of a row is formed in the same order whoever forms it.
template <int DIMV, int U, class Ref, class IdFn, class OutFn>
__device__ __forceinline__ void score_share(const Ref ref, const float* data, uint32_t dim, int metric, uint32_t first, uint32_t count,
                                            int lane, uint32_t member, uint32_t members, IdFn id_of, OutFn out) {
    using Shape = RowShape<DIMV>;
    const int g = Shape::row_of_lane(lane), t = Shape::lane_in_row(lane);
    for (uint32_t base = first + member * Shape::ROWS * U; base < count; base += Shape::ROWS * U * members) {
        RowRegs<DIMV> rows[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            // lane groups past the end re-read the last listed row (same cache lines, no branch); their result is dropped
            const uint32_t idx = base + Shape::ROWS * u + g;
            load_row<DIMV>(rows[u], data + static_cast<size_t>(id_of(idx < count ? idx : count - 1)) * dim, dim, t);
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const uint32_t idx = base + Shape::ROWS * u + g;
            float acc = 0.f;
#pragma unroll
            for (int c = 0; c < Shape::NV; c++) acc = sqdist4(ref.chunk(c, t), rows[u].v[c], acc);
            const float d = finish_distance(row_sum<DIMV>(acc), metric);
            if (t == 0 && idx < count) out(idx, d);
        }
    }
}

template <int DIMV, class IdFn, class OutFn>
__device__ __forceinline__ void score_list(const RowRegs<DIMV>& ref, const float* data, uint32_t dim, int metric,
                                           uint32_t first, uint32_t count, int lane, IdFn id_of, OutFn out) {
    // Steps in flight.  Rows of more than 512 dims are 2-4 KB each and a step holds only two of them: with one step in
    // flight a wavefront had 8 KB on its way, too little to cover the memory latency when a launch has about one
    // wavefront per SIMD (1 000 queries); four steps took the 960-dim beam-512 search from 16.8 to 13.2 ms.
    constexpr int U = DIMV == 8 ? 4 : 2;   // rows of more than 1024 dims (DIMV 16, 32) take 64 registers a lane each: two steps
    score_share<DIMV, U>(RefInRegs<DIMV>{ref}, data, dim, metric, first, count, lane, 0u, 1u, id_of, out);
}

// TEAM: the beam's wavefront is one of several in its workgroup (the others only score rows, see search_team_kernel).
// WHOLE: the host promises beam == MAX_BEAM (asked for beams above 256 only, i.e. beam 512): the two-half merge of such a
// beam needs no lane permutations (merge_beam_full), and the kernel 112 registers instead of 128.
template <int MAX_CAND, int MAX_BEAM, int DIMV, bool TEAM = false, bool WHOLE = false>
struct Beam {
    static_assert(!WHOLE || MAX_BEAM > 256, "beams up to 256 merge in the registers anyway");
    static __device__ __forceinline__ void wave_sync() { wave_sync_in<TEAM>(); }
    static constexpr int NB = MAX_BEAM / 64;
    static constexpr int NC = MAX_CAND / 64;
    static constexpr int NC32 = MAX_CAND / 32;  // items per lane in the reference's 32-lane layout

    float bk[NB];
    uint32_t bv[NB];
    RowRegs<DIMV> q;
    BeamLds<MAX_CAND>* lds;
    uint32_t* hash;
    BeamParams p;
    BeamCounters cnt;
    int lane;
    uint32_t last_scored;   // rows scored by the latest expansion (wave-uniform)

    __device__ __forceinline__ void init(BeamLds<MAX_CAND>* lds_, uint32_t* hash_, const BeamParams& p_, const float* query) {
        lds = lds_;
        hash = hash_;
        p = p_;
        lane = lane_id();
        load_row<DIMV>(q, query, p.dim, RowShape<DIMV>::lane_in_row(lane));
        hash_clear(hash, p.hash_bit, lane);
        wave_sync();
    }

    // One pass of the main loop up to the next expansion's candidate list (what `run` does between two score phases).
    // Returns false when the search is over; otherwise `nv` rows wait to be scored.
    __device__ __forceinline__ bool step_to_list(uint32_t& iter, bool& terminate, const uint32_t* graph, uint32_t self_id, uint32_t& nv) {
        absorb(iter == 0);
        cnt.iterations++;
        const bool reset_now = ((iter + 1) % p.reset_interval) == 0;
        if (reset_now) {
            hash_clear(hash, p.hash_bit, lane);
            wave_sync();
        }
        if (iter + 1 == p.max_iterations) return false;
        const uint32_t parent = select_parent();
        if (parent == kInvalid) terminate = true;
        if (reset_now) {
            restore_hash();
            wave_sync();
        }
        if (terminate && iter >= p.min_iterations) return false;
        nv = expand_list(parent, graph, self_id, kInvalid);
        iter++;
        return true;
    }

    // Expansion of `parent` (reference compute_distance / get_init / result_init second half):
    // every neighbour not yet in the visited set becomes a candidate; `exclude_insert` is never inserted,
    // `exclude_score` is inserted and kept as a candidate id but gets distance FLT_MAX.
    // First half: the candidate slots and the list of slots to score (returns its length).
    __device__ __forceinline__ uint32_t expand_list(uint32_t parent, const uint32_t* graph, uint32_t exclude_insert, uint32_t exclude_score) {
        uint32_t nv = 0;
        if (parent != kInvalid) cnt.graph_rows++;
#pragma unroll
        for (int s0 = 0; s0 < MAX_CAND; s0 += 64) {
            const uint32_t s = s0 + lane;
            uint32_t nid = kInvalid;
            if (s < p.degree && parent != kInvalid) nid = graph[static_cast<size_t>(parent) * p.degree + s];
            const uint32_t flag = (nid != kInvalid && nid != exclude_insert) ? hash_insert(hash, p.hash_bit, nid) : 0;
            const uint32_t cid = flag ? nid : kInvalid;
            lds->cand_id[s] = cid;
            lds->cand_dist[s] = FLT_MAX;
            const bool score = cid != kInvalid && cid != exclude_score;
            const uint64_t m = ballot(score);
            if (score) lds->vlist[nv + prefix_count(m)] = s;
            nv += __popcll(m);
        }
        wave_sync();
        cnt.rows_scored += nv;
        last_scored = nv;
        return nv;
    }

    __device__ __forceinline__ void expand(uint32_t parent, const uint32_t* graph, const float* data,
                                           uint32_t exclude_insert, uint32_t exclude_score) {
        const uint32_t nv = expand_list(parent, graph, exclude_insert, exclude_score);
        BeamLds<MAX_CAND>* l = lds;
        score_list<DIMV>(q, data, p.dim, p.metric, 0, nv, lane,
                         [l](uint32_t idx) { return l->cand_id[l->vlist[idx]]; },
                         [l](uint32_t idx, float d) { l->cand_dist[l->vlist[idx]] = d; });
        wave_sync();
    }

    // Candidate sort, one network over the wavefront (reference sort_for_candidate, single-warp branch,
    // search_kernel.cuh:9-37): strided load, sort, blocked store of every element.
    __device__ __forceinline__ void sort_candidates_one() {
        if constexpr (MAX_CAND == 64) {
            // At most 32 slots in use: the strided load puts them on the even elements of the 64-element network and
            // +inf on the odd ones.  Every comparator of that network then meets at most one real key, or two real
            // keys that the 32-element network compares at the same point of its own sequence and in the same
            // direction, so sorting the 32 slots with the 32-element network gives the same sequence, ties included
            // (the CPU tests compare the two networks on tie-rich inputs), in 15 stages instead of 21.
            // The one exception is a real id whose key is not below FLT_MAX (the build kernels leave the point itself
            // unscored): among the +inf keys its place does depend on the network, so that case takes the long way.
            if (p.degree <= 32) {
                float hk[1];
                uint32_t hv[1];
                const uint32_t slot = lane & 31;   // both halves of the wavefront sort the same 32 slots
                hk[0] = slot < p.degree ? lds->cand_dist[slot] : FLT_MAX;
                hv[0] = slot < p.degree ? lds->cand_id[slot] : kInvalid;
                if (ballot(hv[0] != kInvalid && !(hk[0] < FLT_MAX)) == 0) {
                    WaveNet<32>::sort(hk, hv, lane);
                    wave_sync();
                    lds->cand_dist[lane] = lane < 32 ? hk[0] : FLT_MAX;
                    lds->cand_id[lane] = lane < 32 ? hv[0] : kInvalid;
                    wave_sync();
                    return;
                }
            }
        }
        float ck[NC];
        uint32_t cv[NC];
#pragma unroll
        for (int r = 0; r < NC; r++) {
            const uint32_t e = NC * lane + r;          // element index in the network
            const uint32_t l32 = e / NC32, i = e % NC32;
            const uint32_t slot = l32 + 32 * i;        // reference loads strided: j = lane + 32*i
            ck[r] = slot < p.degree ? lds->cand_dist[slot] : FLT_MAX;
            cv[r] = slot < p.degree ? lds->cand_id[slot] : kInvalid;
        }
        WaveNet<MAX_CAND>::sort(ck, cv, lane);
        wave_sync();
#pragma unroll
        for (int r = 0; r < NC; r++) {
            const uint32_t e = NC * lane + r;
            lds->cand_dist[e] = ck[r];
            lds->cand_id[e] = cv[r];
        }
        wave_sync();
    }

    // Candidate sort for more than 128 slots (reference two-warp branch, search_kernel.cuh:38-94): the two 32-lane
    // halves of the wavefront are the two warps.  Each sorts its half of the slots, a half-cleaner across the halves
    // leaves the smaller keys with half 0, each half merges.  Only slots below min(degree, beam) are defined afterwards.
    __device__ __forceinline__ void sort_candidates_two() {
        constexpr int PER = MAX_CAND / 2, N = PER / 32;
        const uint32_t w = lane >> 5, l = lane & 31;
        float key[N];
        uint32_t val[N];
#pragma unroll
        for (int i = 0; i < N; i++) {
            const uint32_t j = l + 32 * i + PER * w;
            key[i] = j < p.degree ? lds->cand_dist[j] : FLT_MAX;
            val[i] = j < p.degree ? lds->cand_id[j] : kInvalid;
        }
        WaveNet<PER, 32>::sort(key, val, lane);
        wave_sync();
#pragma unroll
        for (int i = 0; i < N; i++) {
            const uint32_t jl = N * l + i, j = jl + PER * w;
            if (j < p.degree && jl < p.beam) {
                lds->cand_dist[j] = key[i];
                lds->cand_id[j] = val[i];
            }
        }
        wave_sync();
        const uint32_t warps_used = (p.beam + PER - 1) / PER;
#pragma unroll
        for (int i = 0; i < N; i++) {
            const uint32_t jl = N * l + i, kl = PER - 1 - jl, j = jl + PER * w, k = MAX_CAND - 1 - j;
            if (w < warps_used && j < p.degree && k < p.degree && kl < p.beam) {
                const float other = lds->cand_dist[k];
                if (key[i] != other && ((w == 0) == (key[i] > other))) {
                    key[i] = other;
                    val[i] = lds->cand_id[k];
                }
            }
        }
        wave_sync();
        WaveNet<PER, 32>::merge(key, val, lane);
#pragma unroll
        for (int i = 0; i < N; i++) {
            const uint32_t jl = N * l + i, j = jl + PER * w;
            if (w < warps_used && j < p.degree && j < p.beam) {
                lds->cand_dist[j] = key[i];
                lds->cand_id[j] = val[i];
            }
        }
        wave_sync();
    }

    // v of the lane 32 places away: one swap of the 32-lane halves of a register pair and a select
    template <class T>
    static __device__ __forceinline__ T other_half(T v, bool upper) {
        const int x = __builtin_bit_cast(int, v);
        const auto s = __builtin_amdgcn_permlane32_swap(x, x, false, false);   // s[0]: upper lanes hold the lower half's, s[1]: the reverse
        return __builtin_bit_cast(T, upper ? s[0] : s[1]);
    }

    // Beam merge for a beam of exactly MAX_BEAM entries (beams above 256; the general form follows).  Element
    // NB * lane + r puts the two halves of the beam into the two 32-lane halves of the wavefront, each in the order its
    // merge network wants, so the compare-exchange between the halves is a swap of register halves; and with
    // half == PER the layout [untouched prefix | padding | touched rest] of a half is the half as it stands, whatever
    // the turning points are, so they are not tracked.
    __device__ __forceinline__ void merge_beam_full() {
        bool replaced = false;
#pragma unroll
        for (int r = 0; r < NB; r++) {
            const uint32_t k = MAX_BEAM - 1 - (NB * lane + r);
            if (k < p.degree) {
                const float c = lds->cand_dist[k];
                if (bk[r] > c) {
                    bk[r] = c;
                    bv[r] = lds->cand_id[k];
                    replaced = true;
                }
            }
        }
        if (ballot(replaced) == 0) return;
        const bool upper = lane >= 32;
#pragma unroll
        for (int r = 0; r < NB; r++) {
            const float ok = other_half(bk[r], upper);
            const uint32_t ov = other_half(bv[r], upper);
            const bool take = upper ? ok > bk[r] : bk[r] > ok;   // entry j of the first half and entry j of the second change places when the first is larger
            bk[r] = take ? ok : bk[r];
            bv[r] = take ? ov : bv[r];
            __builtin_amdgcn_sched_barrier(0);   // one register at a time: interleaved, the eight exchanges cost the kernel a wavefront per SIMD in registers
        }
        WaveNet<MAX_BEAM / 2, 32>::merge(bk, bv, lane);
    }

    // Beam merge for beams above 256 (reference two-warp branch of sort_for_beam, search_kernel.cuh:149-232), on the beam
    // where it sits; beam a multiple of 16, so that a half is whole lanes.  Half 0 of the beam is in lanes [0, H), half 1
    // in lanes [H, 2H) (H = half / NB), pads behind.  The reference's steps, each of which decides where equal keys end
    // up: candidates displace larger entries from the tail (the smallest touched index of each half, its "turning
    // point", is found with a ballot: indices grow with the lane), the halves are compare-exchanged entry by entry (a
    // lane permutation: same register, lane +-H), each 32-lane half of the wavefront gathers its half of the beam as
    // [untouched prefix | padding | touched rest] -- the source of position q is the same register of another lane,
    // because half and PER - half are multiples of NB -- and merges it, and the beam gathers the results back.  Three
    // lane permutations of the beam's registers; the reference copies the beam through shared memory and finds the
    // turning points with atomics.
    __device__ __forceinline__ void merge_beam_general() {
        constexpr int PER = MAX_BEAM / 2;
        constexpr uint32_t kNone = 0xffffffffu;
        const uint32_t half = p.beam / 2, H = half / NB;
        uint32_t first = kNone;            // this lane's smallest element index that a candidate replaced
#pragma unroll
        for (int r = NB - 1; r >= 0; r--) {
            const uint32_t e = NB * lane + r;
            const uint32_t k = p.beam - 1 - e;
            if (e < p.beam && k < p.degree) {
                const float c = lds->cand_dist[k];
                if (bk[r] > c) {
                    bk[r] = c;
                    bv[r] = lds->cand_id[k];
                    first = e;
                }
            }
        }
        const uint64_t touched = ballot(first != kNone);
        if (touched == 0) return;
        const uint64_t lanes0 = (1ull << H) - 1;
        const uint64_t touched0 = touched & lanes0, touched1 = touched >> H;
        const uint32_t t2 = touched0 ? read_lane(first, __builtin_ctzll(touched0)) : half;
        uint32_t t1 = touched1 ? read_lane(first, static_cast<int>(H) + __builtin_ctzll(touched1)) - half : half;

        // the halves against each other: entry j of half 0 and entry j of half 1 change places when the first is larger
        const bool lower = static_cast<uint32_t>(lane) < H, upper = !lower && static_cast<uint32_t>(lane) < 2 * H;
        const int partner = lower ? lane + static_cast<int>(H) : (upper ? lane - static_cast<int>(H) : lane);
        uint32_t moved = kNone;
#pragma unroll
        for (int r = NB - 1; r >= 0; r--) {
            const float ok = shfl_f32(bk[r], partner);
            const uint32_t ov = shfl_u32(bv[r], partner);
            const bool take = lower ? bk[r] > ok : (upper && ok > bk[r]);
            if (take && lower) moved = NB * lane + r;
            bk[r] = take ? ok : bk[r];
            bv[r] = take ? ov : bv[r];
            __builtin_amdgcn_sched_barrier(0);   // one register at a time (interleaved, the permutations of a step hold the beam twice)
        }
        const uint64_t movers = ballot(moved != kNone);
        const uint32_t t0 = movers ? read_lane(moved, __builtin_ctzll(movers)) : half;
        if (t2 < half) t1 = t2;

        // each 32-lane half gathers its half of the beam as [untouched prefix | padding | touched rest]; register i of a
        // position comes from register i of another lane, so the beam's registers are rewritten in place
        const uint32_t w = static_cast<uint32_t>(lane) >> 5, l = static_cast<uint32_t>(lane) & 31;
        const uint32_t turning = w ? t1 : t0;
        const uint32_t gap = PER - half;                       // the rest sits `gap` positions further on
        const int from_prefix = static_cast<int>(l + H * w), from_rest = static_cast<int>(l + H * w) - static_cast<int>(gap / NB);
#pragma unroll
        for (int i = 0; i < NB; i++) {
            const uint32_t q = NB * l + i;
            const bool in_prefix = q < turning;
            const bool in_rest = q >= gap && q - gap >= turning;     // q - gap < half holds for every q < PER
            const int src = in_prefix ? from_prefix : (in_rest ? from_rest : lane);
            const float k = shfl_f32(bk[i], src);
            const uint32_t v = shfl_u32(bv[i], src);
            bk[i] = in_prefix || in_rest ? k : FLT_MAX;
            bv[i] = in_prefix || in_rest ? v : kInvalid;
            __builtin_amdgcn_sched_barrier(0);
        }
        WaveNet<PER, 32>::merge(bk, bv, lane);
        // back into beam order: the first `half` positions of half-wave w are elements [half * w, half * w + half)
        const uint32_t w2 = static_cast<uint32_t>(lane) >= H ? 1u : 0u;
        const int back = static_cast<int>(static_cast<uint32_t>(lane) - H * w2 + 32 * w2) & 63;
        const bool live = static_cast<uint32_t>(lane) < 2 * H;
#pragma unroll
        for (int r = 0; r < NB; r++) {
            const float k = shfl_f32(bk[r], back);
            const uint32_t v = shfl_u32(bv[r], back);
            bk[r] = live ? k : FLT_MAX;
            bv[r] = live ? v : kInvalid;
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // The candidates of the latest expansion that are below the last beam entry, as a lane mask (one candidate slot per
    // lane).  None: the beam stays as it is -- the half-cleaner of the merge replaces an entry only by a strictly smaller
    // candidate, entry `beam - 1 - k` by the k-th smallest, so if even the smallest candidate is not below the largest
    // entry nothing is replaced, and the candidate sort in front of it only feeds that test.  Half of all iterations of
    // a wide beam end here (the further a search has come, the fewer neighbours of its frontier are nearer than the worst
    // entry it holds), for one LDS read per lane.
    __device__ __forceinline__ uint64_t entering(float& ck) {
        static_assert(MAX_CAND == 64, "one candidate slot per lane");
        // The beam is ascending, so its last entry is the largest key of the lane that holds it among that lane's entries
        // below `beam` (written as a maximum: a chain of selects between the registers becomes a run-time index, which
        // moves the beam out of the registers).  Keys are not negative.
        const uint32_t last = p.beam - 1;
        float tail;
        if (p.beam == MAX_BEAM) {   // a beam that fills its bucket ends in the last register of the last lane
            tail = read_lane(bk[NB - 1], 63);
        } else {
            float mine = bk[0];
#pragma unroll
            for (int r = 1; r < NB; r++) mine = fmaxf(mine, NB * lane + r <= static_cast<int>(last) ? bk[r] : 0.f);
            tail = read_lane(mine, static_cast<int>(last / NB));
        }
        ck = static_cast<uint32_t>(lane) < p.degree ? lds->cand_dist[lane] : FLT_MAX;
        return ballot(ck < tail);
    }

    // reference update_result_buffer: sort the candidates, then fold them into the beam
    __device__ __forceinline__ void absorb(bool first) {
        // No row scored: every candidate distance is FLT_MAX, the sort would not move anything (equal keys are never
        // exchanged) and no candidate can displace a beam entry, so the beam stays as it is.
        if (!first && last_scored == 0) return;
        if constexpr (MAX_CAND == 64) {
            if (!first) {
                float ck;
                const uint64_t em = entering(ck);
                if (em == 0) return;
            }
        }
        if constexpr (MAX_CAND > 128) sort_candidates_two();
        else sort_candidates_one();
        if (first) {
#pragma unroll
            for (int r = 0; r < NB; r++) {
                const uint32_t e = NB * lane + r;
                const bool take = e < p.beam && e < p.degree;
                bk[r] = take ? lds->cand_dist[e] : FLT_MAX;
                bv[r] = take ? lds->cand_id[e] : kInvalid;
            }
        } else if constexpr (MAX_BEAM > 256) {
            if constexpr (WHOLE) merge_beam_full();
            else merge_beam_general();
        } else {
            bool replaced = false;
#pragma unroll
            for (int r = 0; r < NB; r++) {
                const uint32_t e = NB * lane + r;
                const uint32_t k = MAX_BEAM - 1 - e;
                if (k < p.beam && k < p.degree) {
                    const float c = lds->cand_dist[k];
                    if (bk[r] > c) {
                        bk[r] = c;
                        bv[r] = lds->cand_id[k];
                        replaced = true;
                    }
                }
            }
            // Nothing replaced: the beam is still the ascending sequence the previous merge left, and the merge
            // network (strict comparisons) is the identity on it.
            if (ballot(replaced) != 0) {
                WaveNet<MAX_BEAM>::merge(bk, bv, lane);
                if (p.beam < MAX_BEAM) {   // a beam that fills its bucket has nothing behind it (and the lane masks of this loop are not held)
#pragma unroll
                    for (int r = 0; r < NB; r++) {
                        const uint32_t e = NB * lane + r;
                        if (e >= p.beam) {
                            bk[r] = FLT_MAX;
                            bv[r] = kInvalid;
                        }
                    }
                }
            }
        }
        wave_sync();
    }

    // first unexplored beam entry (reference select_current_point); marks it explored
    __device__ __forceinline__ uint32_t select_parent() {
        // entries behind the beam are pads (kInvalid), which carry the explored bit like every unfilled entry
        int rsel = NB;
#pragma unroll
        for (int r = NB - 1; r >= 0; r--)
            if ((bv[r] & kExplored) == 0) rsel = r;
        const uint64_t m = ballot(rsel < NB);
        if (m == 0) return kInvalid;
        const int src = __builtin_ctzll(m);
        const int r_src = __builtin_amdgcn_readlane(rsel, src);
        uint32_t mine = 0;
#pragma unroll
        for (int r = 0; r < NB; r++) {
            if (r == r_src) {
                mine = bv[r];
                if (lane == src) bv[r] |= kExplored;
            }
        }
        return read_lane(mine, src);
    }

    __device__ __forceinline__ void restore_hash() {
#pragma unroll
        for (int r = 0; r < NB; r++) {
            const uint32_t e = NB * lane + r;
            if (e < p.beam) hash_insert(hash, p.hash_bit, bv[r] & kClean);
        }
    }

    // main loop; candidates of the entry expansion must already be in LDS
    __device__ __forceinline__ void run(const uint32_t* graph, const float* data, uint32_t self_id) {
        uint32_t iter = 0;
        bool terminate = false;
        while (true) {
            absorb(iter == 0);
            cnt.iterations++;
            const bool reset_now = ((iter + 1) % p.reset_interval) == 0;
            if (reset_now) {
                hash_clear(hash, p.hash_bit, lane);
                wave_sync();
            }
            if (iter + 1 == p.max_iterations) break;
            const uint32_t parent = select_parent();
            if (parent == kInvalid) terminate = true;
            if (reset_now) {
                restore_hash();
                wave_sync();
            }
            if (terminate && iter >= p.min_iterations) break;
            expand(parent, graph, data, self_id, kInvalid);
            iter++;
        }
    }

    // `counters` holds kCounterStripes x 3 u64 (striped by workgroup: a single shared address would serialise the
    // whole launch); the host adds the stripes up
    __device__ __forceinline__ void flush_counters(unsigned long long* counters) {
        if (counters != nullptr && lane == 0) {
            unsigned long long* slot = counters + 3 * (blockIdx.x % kCounterStripes);
            atomicAdd(&slot[0], static_cast<unsigned long long>(cnt.iterations));
            atomicAdd(&slot[1], static_cast<unsigned long long>(cnt.rows_scored));
            atomicAdd(&slot[2], static_cast<unsigned long long>(cnt.graph_rows));
        }
    }
};

// Nearest centroid by the reference's sort network (search_kernel.cuh:259-268, distance.cuh:29-60):
// strided load, blocked store, element 0 is the winner.  One wavefront; scratch holds `centroid_num` pairs.
template <int MAX_CENTROID, int DIMV, bool TEAM = false>
__device__ __forceinline__ uint32_t nearest_centroid(const RowRegs<DIMV>& q, const float* centroids, uint32_t centroid_num,
                                                     uint32_t dim, int metric, float* cent_dist, int lane) {
    using Shape = RowShape<DIMV>;
    const int g = Shape::row_of_lane(lane), t = Shape::lane_in_row(lane);
    for (uint32_t c0 = 0; c0 < centroid_num; c0 += Shape::ROWS) {
        const uint32_t c = c0 + g;
        RowRegs<DIMV> row;
        if (c < centroid_num) {
            load_row<DIMV>(row, centroids + static_cast<size_t>(c) * dim, dim, t);
        } else {
            row = q;
        }
        const float d = finish_distance(row_sum<DIMV>(partial_sqdist<DIMV>(q, row)), metric);
        if (t == 0 && c < centroid_num) cent_dist[c] = d;
    }
    wave_sync_in<TEAM>();
    constexpr int NR = WaveNet<MAX_CENTROID>::NR;
    constexpr int N32 = MAX_CENTROID / 32;
    float k[NR];
    uint32_t v[NR];
#pragma unroll
    for (int r = 0; r < NR; r++) {
        const uint32_t e = NR * lane + r;
        const uint32_t j = (e / N32) + 32 * (e % N32);
        const bool ok = (MAX_CENTROID >= 64 || lane < 32) && j < centroid_num;
        k[r] = ok ? cent_dist[j] : FLT_MAX;
        v[r] = ok ? j : kInvalid;
    }
    WaveNet<MAX_CENTROID>::sort(k, v, lane);
    wave_sync_in<TEAM>();
    return read_lane(v[0], 0);
}

}  // namespace glide
