// Bitonic sort / merge of (float key, u32 value) pairs held in the registers of one 64-lane wavefront.
//
// The reference (bitonic.cuh:24-212) runs the standard bitonic network over M = 32*N elements with element
// index e = N*lane32 + i and a compare-exchange that does nothing on equal keys.  The network is a property of
// the element indices, not of the lane width, so the same comparator sequence is executed here with
// e = NR*lane64 + r, NR = M/64 (M = 32 uses lanes 0..31 with NR = 1; lanes 32..63 run a private copy).
// Same comparators in the same stage order => identical output sequence, ties included.
// With LANES = 32 the two halves of the wavefront run two independent networks of M elements each (NR = M/32):
// the reference's two-warp variants, one warp per half.
#pragma once
#include "common.hpp"

namespace glide {

template <int M, int LANES = (M >= 64 ? 64 : 32)>
struct WaveNet {
    static_assert(M == 32 || M == 64 || M == 128 || M == 256 || M == 512, "network size");
    static_assert((LANES == 64 || LANES == 32) && M >= LANES, "lanes per network");
    static constexpr int NR = M / LANES;

    // compare-exchange of two registers of the same lane (bitonic.cuh:25-34)
    static __device__ __forceinline__ void cmpx_reg(float& k0, uint32_t& v0, float& k1, uint32_t& v1, bool asc) {
        if ((k0 != k1) && ((k0 < k1) != asc)) {
            float tk = k0; k0 = k1; k1 = tk;
            uint32_t tv = v0; v0 = v1; v1 = tv;
        }
    }
    // Lanes that keep the smaller key in stage (K, J) for register r: bit l set <=> lane l is the lower partner of an
    // ascending pair or the upper partner of a descending one.  A compile-time constant.
    template <int K, int J>
    static constexpr uint64_t keep_min_mask(int r) {
        constexpr int LM = J / NR;
        uint64_t m = 0;
        for (int l = 0; l < 64; l++) {
            const int e = NR * (l % LANES) + r;
            const bool asc = (K >= M) ? true : ((e & K) == 0);
            const bool lower = (l & LM) == 0;
            if (lower == asc) m |= 1ull << l;
        }
        return m;
    }
    // compare-exchange with the lane `lane ^ LM` (bitonic.cuh:36-44): a lane that keeps the minimum takes the partner's
    // pair iff partner < mine, a lane that keeps the maximum iff mine < partner.  Both tests are strict, so equal keys
    // are never exchanged (the reference's k0 != k1 guard).  The two predicates are combined with the constant
    // keep-min mask on the scalar unit; for the half-swap (LM = 32) the second predicate is the first with its halves
    // swapped, which costs no vector instruction.  (The scalar unit is shared by the four SIMDs of a CU, so longer
    // scalar sequences that would save the second compare for the other distances do not pay.)
    template <int LM>
    static __device__ __forceinline__ void cmpx_lane(float& k, uint32_t& v, uint64_t keep_min) {
        const float ok = lane_xor<LM>(k);
        const uint32_t ov = lane_xor<LM>(v);
        const uint64_t less = __builtin_amdgcn_ballot_w64(ok < k);
        const uint64_t more = LM == 32 ? mask_xor<32>(less) : __builtin_amdgcn_ballot_w64(k < ok);
        const uint64_t take = (less & keep_min) | (more & ~keep_min);
        k = select_by_mask(k, ok, take);
        v = select_by_mask(v, ov, take);
    }

    // one network stage: partner distance J (elements), direction block K (elements); K == M means all ascending
    template <int K, int J>
    static __device__ __forceinline__ void stage(float (&k)[NR], uint32_t (&v)[NR], int lane) {
        if constexpr (J < NR) {
#pragma unroll
            for (int r = 0; r < NR; r++) {
                if ((r & J) == 0) {
                    const int e = NR * (lane % LANES) + r;
                    const bool asc = (K >= M) ? true : ((e & K) == 0);
                    cmpx_reg(k[r], v[r], k[r | J], v[r | J], asc);
                }
            }
        } else {
            constexpr int LM = J / NR;
#pragma unroll
            for (int r = 0; r < NR; r++) cmpx_lane<LM>(k[r], v[r], keep_min_mask<K, J>(r));
        }
    }

    template <int K, int J>
    static __device__ __forceinline__ void merge_from(float (&k)[NR], uint32_t (&v)[NR], int lane) {
        stage<K, J>(k, v, lane);
        if constexpr (J > 1) merge_from<K, J / 2>(k, v, lane);
    }
    template <int K>
    static __device__ __forceinline__ void sort_from(float (&k)[NR], uint32_t (&v)[NR], int lane) {
        merge_from<K, K / 2>(k, v, lane);
        if constexpr (K < M) sort_from<K * 2>(k, v, lane);
    }

    // full ascending sort (reference warp_sort, bitonic.cuh:207-212)
    static __device__ __forceinline__ void sort(float (&k)[NR], uint32_t (&v)[NR], int lane) { sort_from<2>(k, v, lane); }
    // final ascending merge of a bitonic sequence (reference warp_merge with range 32, bitonic.cuh:202-205)
    static __device__ __forceinline__ void merge(float (&k)[NR], uint32_t (&v)[NR], int lane) { merge_from<M, M / 2>(k, v, lane); }
};

}  // namespace glide
