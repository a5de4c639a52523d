// Wave64 device primitives shared by every GLIDE kernel on gfx950 (CDNA4).
//
// One wavefront = 64 lanes.  All per-item kernels (search, sub-graph build, refine) give one item to one
// wavefront, so the "warp 0 / other warps" split and the block barriers of the reference collapse into
// straight-line wave code.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <float.h>

namespace glide {

constexpr uint32_t kInvalid = 0xffffffffu;
constexpr uint32_t kExplored = 0x80000000u;  // reference utils.cuh:5-8
constexpr uint32_t kClean = 0x7fffffffu;
constexpr int kWave = 64;

enum Metric : int { kEuclidean = 0, kCosine = 1 };  // reference params.cuh:5-8

__host__ __device__ constexpr uint32_t round_up32(uint32_t p) { return (p + 31u) & ~31u; }  // utils.cuh:21-23
// a / b rounded up, without the wrap of (a + b - 1) when a is within b of 2^32
__host__ __device__ constexpr uint32_t ceil_div(uint32_t a, uint32_t b) { return a / b + (a % b != 0); }

__device__ __forceinline__ int lane_id() { return static_cast<int>(__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u))); }

// ---------------------------------------------------------------- cross-lane exchange, compile-time xor mask
// xor 1,2: DPP quad_perm; xor 4: two banked DPP row shifts; xor 8: DPP row_ror:8; xor 16: ds_swizzle (LDS
// crossbar, no memory); xor 32: ds_bpermute.
template <int MASK>
__device__ __forceinline__ int lane_xor_i(int v) {
    static_assert(MASK == 1 || MASK == 2 || MASK == 4 || MASK == 8 || MASK == 16 || MASK == 32, "xor mask");
    // mov_dpp leaves the destination's previous value undefined for lanes the pattern does not write; every pattern
    // below writes all 64 lanes, so no register has to be initialised first
    if constexpr (MASK == 1) {
        return __builtin_amdgcn_mov_dpp(v, 0xB1, 0xf, 0xf, false);  // quad_perm:[1,0,3,2]
    } else if constexpr (MASK == 2) {
        return __builtin_amdgcn_mov_dpp(v, 0x4E, 0xf, 0xf, false);  // quad_perm:[2,3,0,1]
    } else if constexpr (MASK == 4) {
        int r = __builtin_amdgcn_mov_dpp(v, 0x104, 0xf, 0x5, false);    // row_shl:4 -> banks 0,2 read lane+4
        r = __builtin_amdgcn_update_dpp(r, v, 0x114, 0xf, 0xA, false);  // row_shr:4 -> banks 1,3 read lane-4
        return r;
    } else if constexpr (MASK == 8) {
        return __builtin_amdgcn_mov_dpp(v, 0x128, 0xf, 0xf, false);  // row_ror:8
    } else if constexpr (MASK == 16) {
        return __builtin_amdgcn_ds_swizzle(v, 0x401F);  // BITMODE and=0x1f or=0 xor=0x10
    } else {
        return __builtin_amdgcn_ds_bpermute((lane_id() ^ 32) << 2, v);
    }
}
// A 64-lane predicate mask with every bit moved to the lane MASK away (the partner's predicate), on the scalar unit.
template <int MASK>
__device__ __forceinline__ uint64_t mask_xor(uint64_t m) {
    constexpr uint64_t low = MASK == 1 ? 0x5555555555555555ull : MASK == 2 ? 0x3333333333333333ull : MASK == 4 ? 0x0F0F0F0F0F0F0F0Full
                           : MASK == 8 ? 0x00FF00FF00FF00FFull : MASK == 16 ? 0x0000FFFF0000FFFFull : 0x00000000FFFFFFFFull;
    return ((m & low) << MASK) | ((m >> MASK) & low);
}
// per-lane select driven by a scalar 64-bit mask: lane l gets `b` where bit l is set, else `a`
__device__ __forceinline__ float select_by_mask(float a, float b, uint64_t mask) {
    float out;
    asm("v_cndmask_b32_e64 %0, %1, %2, %3" : "=v"(out) : "v"(a), "v"(b), "s"(mask));
    return out;
}
__device__ __forceinline__ uint32_t select_by_mask(uint32_t a, uint32_t b, uint64_t mask) {
    uint32_t out;
    asm("v_cndmask_b32_e64 %0, %1, %2, %3" : "=v"(out) : "v"(a), "v"(b), "s"(mask));
    return out;
}
template <int MASK>
__device__ __forceinline__ float lane_xor(float v) { return __builtin_bit_cast(float, lane_xor_i<MASK>(__builtin_bit_cast(int, v))); }
template <int MASK>
__device__ __forceinline__ uint32_t lane_xor(uint32_t v) { return static_cast<uint32_t>(lane_xor_i<MASK>(static_cast<int>(v))); }

__device__ __forceinline__ float read_lane(float v, int lane) { return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane)); }
__device__ __forceinline__ uint32_t read_lane(uint32_t v, int lane) { return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), lane)); }
__device__ __forceinline__ uint32_t shfl_u32(uint32_t v, int src_lane) { return static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(src_lane << 2, static_cast<int>(v))); }
__device__ __forceinline__ float shfl_f32(float v, int src_lane) { return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(src_lane << 2, __builtin_bit_cast(int, v))); }

__device__ __forceinline__ uint64_t ballot(bool p) { return __ballot(p); }
// number of set bits of `mask` strictly below this lane
__device__ __forceinline__ uint32_t prefix_count(uint64_t mask) {
    return __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(mask >> 32), __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), 0u));
}

// Sum over each 32-lane half of the wave; every lane of a half ends with that half's total.
__device__ __forceinline__ float half_wave_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, false));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, false));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, false));  // row_half_mirror
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xf, 0xf, false));  // row_mirror
    v += lane_xor<16>(v);
    return v;
}
// Sum over the whole wave; every lane ends with the total.
__device__ __forceinline__ float wave_sum(float v) {
    v = half_wave_sum(v);
    v += lane_xor<32>(v);
    return v;
}

// Prefix sum over the 64 lanes without LDS traffic: four shifted adds inside each row of 16 lanes, then lane 15 of a row
// is added to the next row (rows 1 and 3) and lane 31 to the upper half (rows 2 and 3).  Lanes a step does not feed add 0.
__device__ __forceinline__ uint32_t wave_exclusive_scan(uint32_t value, uint32_t& total) {
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

// ---------------------------------------------------------------- LDS open-addressing hash set (reference hashmap.cuh:23-56)
__device__ __forceinline__ void hash_clear(uint32_t* table, uint32_t bitlen, int lane) {
    for (uint32_t i = lane; i < (1u << bitlen); i += kWave) table[i] = kInvalid;
}
// returns 1 iff `key` was newly stored; 0 if present or the table is full
__device__ __forceinline__ uint32_t hash_insert(uint32_t* table, uint32_t bitlen, uint32_t key) {
    const uint32_t size = 1u << bitlen;
    const uint32_t mask = size - 1;
    uint32_t index = (key ^ (key >> bitlen)) & mask;
    for (uint32_t i = 0; i < size; i++) {
        const uint32_t old = atomicCAS(&table[index], kInvalid, key);
        if (old == kInvalid) return 1;
        if (old == key) return 0;
        index = (index + 1) & mask;
    }
    return 0;
}

// ---------------------------------------------------------------- row distance, several rows per wave-wide load
// A row is read by a group of LPR adjacent lanes, 16 bytes per lane and load, NV loads per lane; lane t of a group
// owns dims [(c*LPR + t)*4, +4) of load c, so one load instruction touches LPR*16 contiguous bytes of each row.
// Narrow rows use narrow groups: the cross-lane sum then needs log2(LPR) steps instead of 5 and one instruction
// serves 64/LPR rows.  DIMV selects the shape by row length (dim <= 128*DIMV):
//   DIMV 1: 8 lanes x 4 loads (8 rows per wavefront)    DIMV 2: 16 lanes x 4 loads (4 rows)
//   DIMV 4: 32 lanes x 4 loads (2 rows)                 DIMV 8 / 16: 32 lanes x 8 / 16 loads (2 rows)
//   DIMV 32: 64 lanes x 16 loads (1 row; up to 4096 dims)
template <int DIMV>
struct RowShape {
    static_assert(DIMV == 1 || DIMV == 2 || DIMV == 4 || DIMV == 8 || DIMV == 16 || DIMV == 32, "row shape");
    static constexpr int LPR = DIMV == 1 ? 8 : (DIMV == 2 ? 16 : (DIMV == 32 ? 64 : 32));
    static constexpr int NV = DIMV >= 16 ? 16 : (DIMV == 8 ? 8 : 4);
    static constexpr int ROWS = 64 / LPR;
    static __device__ __forceinline__ int lane_in_row(int lane) { return lane & (LPR - 1); }
    static __device__ __forceinline__ int row_of_lane(int lane) { return lane / LPR; }
};

template <int DIMV>
struct RowRegs {
    float4 v[RowShape<DIMV>::NV];
};

// t = RowShape<DIMV>::lane_in_row(lane)
template <int DIMV>
__device__ __forceinline__ void load_row(RowRegs<DIMV>& r, const float* row, uint32_t dim, int t) {
#pragma unroll
    for (int c = 0; c < RowShape<DIMV>::NV; c++) {
        const uint32_t d0 = (c * RowShape<DIMV>::LPR + t) * 4;
        r.v[c] = d0 < dim ? *reinterpret_cast<const float4*>(row + d0) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
}

__device__ __forceinline__ float sqdist4(const float4& a, const float4& b, float acc) {
    const float dx = a.x - b.x, dy = a.y - b.y, dz = a.z - b.z, dw = a.w - b.w;
    acc = fmaf(dx, dx, acc);
    acc = fmaf(dy, dy, acc);
    acc = fmaf(dz, dz, acc);
    acc = fmaf(dw, dw, acc);
    return acc;
}

template <int DIMV>
__device__ __forceinline__ float partial_sqdist(const RowRegs<DIMV>& a, const RowRegs<DIMV>& b) {
    float acc = 0.f;
#pragma unroll
    for (int c = 0; c < RowShape<DIMV>::NV; c++) acc = sqdist4(a.v[c], b.v[c], acc);
    return acc;
}

// Sum over each group of LPR lanes; every lane of a group ends with the group's total.
template <int DIMV>
__device__ __forceinline__ float row_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, false));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, false));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, false));  // row_half_mirror
    if constexpr (RowShape<DIMV>::LPR >= 16)
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xf, 0xf, false));  // row_mirror
    if constexpr (RowShape<DIMV>::LPR >= 32) v += lane_xor<16>(v);
    if constexpr (RowShape<DIMV>::LPR >= 64) v += lane_xor<32>(v);
    return v;
}

// reference distance.cuh:22-26: Euclidean reports sqrt, Cosine the squared L2 of pre-normalised rows
__device__ __forceinline__ float finish_distance(float sq, int metric) { return metric == kEuclidean ? sqrtf(sq) : sq; }

}  // namespace glide
