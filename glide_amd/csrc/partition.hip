// Locality partitioning: point -> centroid assignment (fp32 MFMA tile + norm-trick ranking, exact distances to the
// centroids within the ranking's error band of the second best), stable slot numbering, row reordering, row sampling and a small Lloyd k-means.
// Reference: define_partition_kernel (partition_kernel.cuh:22-66), reorder_kernel (:68-100), sample_kernel
// (:7-20), host sequencing partition.cuh:8-193.
#include "common.hpp"
#include "host_util.hpp"
#include <mutex>

namespace glide {

typedef float float16v __attribute__((ext_vector_type(16)));

constexpr int kTilePoints = 128;   // points per workgroup (4 wavefronts x 32)
constexpr int kChunk = 32;         // dims staged per step
constexpr int kLdsStride = 36;     // floats per staged row (32 + 4 pad keeps 16-byte alignment, spreads banks)

struct AssignArgs {
    const float* data;
    const float* centroids;
    const float* centroid_norms;   // ||c||^2, fp32
    uint32_t* segment_indexes;     // num x 3: segment, (slot filled later), boundary flag as 0 / 0xffffffff
    uint32_t* tile_hist;           // (C + 1) x tiles: bin-major, so that the scan over tiles reads each bin as one run
    float* nearest_dists;          // num x 2 or null
    uint32_t num, dim, centroid_num;
    float boundary_factor;
    int metric;
};

// exact distance of one point row to one centroid, one 32-lane half per pair (same arithmetic as the search kernels)
__device__ __forceinline__ float exact_distance_half(const float* x, const float* c, uint32_t dim, int t) {
    float acc = 0.f;
    for (uint32_t d0 = t * 4; d0 < dim; d0 += 128) {
        const float4 a = *reinterpret_cast<const float4*>(x + d0);
        const float4 b = *reinterpret_cast<const float4*>(c + d0);
        float dx = a.x - b.x, dy = a.y - b.y, dz = a.z - b.z, dw = a.w - b.w;
        acc = fmaf(dx, dx, acc);
        acc = fmaf(dy, dy, acc);
        acc = fmaf(dz, dz, acc);
        acc = fmaf(dw, dw, acc);
    }
    return half_wave_sum(acc);
}

// Ranking pass of assign_kernel: which centroids have to be measured exactly.
// The matrix cores give s(c) = ||c||^2 - 2 x.c, which ranks the centroids of one point like the squared distance but
// carries rounding error.  With E bounding |s(c) + ||x||^2 - D(c)| for the distance D(c) that the exact pass computes
// (squared, before the root), a centroid among the two nearest by D has s(c) <= s2 + 2 E, s2 being the second smallest
// score: were it larger, two other centroids would have scores below s(c) - 2 E and therefore smaller D.  So the
// centroids within `band` = 2 E of the second smallest score are the only ones the exact pass has to see -- two of
// them for nearly every point -- and the nearest two come out as if every centroid had been measured.
// E: the dot product of dim terms is off by at most (dim + 2) u (||x||^2 + ||c||^2) / 2 whatever the order of its sums
// (u = 2^-24; doubled here in case the matrix pipeline rounds products and sums separately), ||c||^2 as stored by
// (dim + 6) u ||c||^2, the final multiply-add by u |s|, D by (dim + 2) u D <= 2 (dim + 2) u (||x||^2 + ||c||^2), and
// roots of D within 3 u of each other may tie: together below 6 (2 dim + 16) u (||x||^2 + max ||c||^2).
__device__ __forceinline__ float assign_band(uint32_t dim, float x_norm, float max_centroid_norm) {
    return 12.f * static_cast<float>(2 * dim + 16) * 5.9604645e-8f * 1.01f * (x_norm + max_centroid_norm);
}

constexpr int kKeep = 4;   // candidates one lane can pass to the exact pass; a point with more is measured against every centroid

// smallest two of a point's candidates by (distance, centroid id)
__device__ __forceinline__ void nearest_two(float dk, uint32_t ck, float& d0, uint32_t& c0, float& d1, uint32_t& c1) {
    const bool lt0 = dk < d0 || (dk == d0 && ck < c0);
    const bool lt1 = dk < d1 || (dk == d1 && ck < c1);
    if (lt0) {
        d1 = d0; c1 = c0;
        d0 = dk; c0 = ck;
    } else if (lt1) {
        d1 = dk; c1 = ck;
    }
}

// CB = number of 32-centroid row blocks held in accumulators (centroid_num <= 32*CB).
// One wavefront owns 32 points.  The matrix instruction takes the centroids as its A operand and the points as B, so
// lane (t, half) ends with the scores of point t against 16 centroids of every block in its own registers and ranks
// them there: no score tile, no barrier after the matrix passes.
// At least two wavefronts per SIMD: with eight blocks the 128 accumulators leave 128 registers for everything else, and
// a second wavefront is what keeps the matrix cores fed while the first one ranks and measures.
template <int CB>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void assign_kernel(AssignArgs a) {
    extern __shared__ __align__(16) float smem[];
    float* cent_tile = smem;                                   // [32*CB][kLdsStride]
    float* x_tile = cent_tile + 32 * CB * kLdsStride;          // [4 waves][32][kLdsStride]
    float* cnorm = x_tile + 4 * 32 * kLdsStride;               // [32*CB]: ||c||^2, +inf beyond centroid_num
    uint32_t* hist = reinterpret_cast<uint32_t*>(cnorm + 32 * CB);   // [C + 1]

    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int half = lane >> 5, t = lane & 31;
    const uint32_t tile_base = blockIdx.x * kTilePoints;
    const uint32_t wave_base = tile_base + wave * 32;
    float* xw = x_tile + wave * 32 * kLdsStride;

    for (uint32_t i = threadIdx.x; i <= a.centroid_num; i += 256) hist[i] = 0;
    for (uint32_t i = threadIdx.x; i < 32 * CB; i += 256) cnorm[i] = i < a.centroid_num ? a.centroid_norms[i] : __builtin_inff();

    float16v acc[CB];
#pragma unroll
    for (int cb = 0; cb < CB; cb++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[cb][r] = 0.f;

    // Chunks of kChunk dims go global -> registers -> LDS; the loads of chunk k+1 are issued before the matrix
    // instructions of chunk k, so their latency is covered by the MFMA work.  The squared norms of the points (for the
    // error band of the ranking) are summed on the way.
    float4 cpre[CB], xpre[4];
    float xsq[4] = {0.f, 0.f, 0.f, 0.f};
    auto prefetch = [&](uint32_t k0) {
#pragma unroll
        for (int it = 0; it < CB; it++) {   // centroid chunk: 8 lanes x float4 per row, 32*CB rows over 256 threads
            const uint32_t idx = threadIdx.x + 256 * it;
            const uint32_t row = idx >> 3, d0 = k0 + (idx & 7) * 4;
            cpre[it] = (row < a.centroid_num && d0 < a.dim) ? *reinterpret_cast<const float4*>(a.centroids + static_cast<size_t>(row) * a.dim + d0)
                                                           : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int it = 0; it < 4; it++) {    // this wave's 32 points
            const uint32_t row = it * 8 + (lane >> 3);
            const uint32_t p = wave_base + row, d0 = k0 + (lane & 7) * 4;
            xpre[it] = (p < a.num && d0 < a.dim) ? *reinterpret_cast<const float4*>(a.data + static_cast<size_t>(p) * a.dim + d0)
                                                 : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    prefetch(0);
    for (uint32_t k0 = 0; k0 < a.dim; k0 += kChunk) {
        __syncthreads();   // every wave is done with the previous chunk
#pragma unroll
        for (int it = 0; it < CB; it++) {
            const uint32_t idx = threadIdx.x + 256 * it;
            *reinterpret_cast<float4*>(cent_tile + (idx >> 3) * kLdsStride + (idx & 7) * 4) = cpre[it];
        }
#pragma unroll
        for (int it = 0; it < 4; it++) {
            *reinterpret_cast<float4*>(xw + (it * 8 + (lane >> 3)) * kLdsStride + (lane & 7) * 4) = xpre[it];
            xsq[it] = fmaf(xpre[it].x, xpre[it].x, fmaf(xpre[it].y, xpre[it].y, fmaf(xpre[it].z, xpre[it].z, fmaf(xpre[it].w, xpre[it].w, xsq[it]))));
        }
        __syncthreads();
        if (k0 + kChunk < a.dim) prefetch(k0 + kChunk);
        // v_mfma_f32_32x32x2_f32: lane supplies A[i = lane%32][k-slot = lane/32] and B[k-slot][j = lane%32].
        // A k-slot pair is fed from one float4 per half (dims kk+4*half .. +3), component by component.
#pragma unroll
        for (int kk = 0; kk < kChunk; kk += 8) {
            const float4 xv = *reinterpret_cast<const float4*>(xw + t * kLdsStride + kk + 4 * half);
#pragma unroll
            for (int cb = 0; cb < CB; cb++) {
                const float4 cv = *reinterpret_cast<const float4*>(cent_tile + (cb * 32 + t) * kLdsStride + kk + 4 * half);
                acc[cb] = __builtin_amdgcn_mfma_f32_32x32x2f32(cv.x, xv.x, acc[cb], 0, 0, 0);
                acc[cb] = __builtin_amdgcn_mfma_f32_32x32x2f32(cv.y, xv.y, acc[cb], 0, 0, 0);
                acc[cb] = __builtin_amdgcn_mfma_f32_32x32x2f32(cv.z, xv.z, acc[cb], 0, 0, 0);
                acc[cb] = __builtin_amdgcn_mfma_f32_32x32x2f32(cv.w, xv.w, acc[cb], 0, 0, 0);
            }
        }
    }

    // From here on the wavefront is on its own.  Its x tile is free (LDS operations of one wavefront complete in order,
    // and the last matrix pass has read it) and becomes its scratch:
    uint32_t* cand_by_lane = reinterpret_cast<uint32_t*>(xw);      // [64][kKeep] centroids within the band, per lane
    uint32_t* lane_first = cand_by_lane + 64 * kKeep;              // [64] where a lane's pairs start
    uint32_t* lane_pairs = lane_first + 64;                        // [64] how many it has
    uint32_t* pairs = lane_pairs + 64;                             // [64 * kKeep] (point << 16 | centroid), one per exact distance
    float* exact = reinterpret_cast<float*>(pairs + 64 * kKeep);   // [64 * kKeep]
    float* x_norm = exact + 64 * kKeep;                            // [32]
    static_assert(64 * kKeep * 3 + 128 + 32 <= 32 * kLdsStride, "scratch fits the x tile");
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const float total = row_sum<1>(xsq[it]);   // the 8 lanes that staged a row
        if ((lane & 7) == 0) x_norm[it * 8 + (lane >> 3)] = total;
    }
    float max_cn = 0.f;
    for (uint32_t i = lane; i < a.centroid_num; i += 64) max_cn = fmaxf(max_cn, cnorm[i]);
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) max_cn = fmaxf(max_cn, __shfl_xor(max_cn, m));
    __builtin_amdgcn_wave_barrier();

    // ---- ranking, first sweep: score = ||c||^2 - 2 x.c and the two smallest scores of the point.  The scores are not
    // kept (a second copy of every accumulator would halve the wavefronts a SIMD holds): the second sweep forms them again.
    // Accumulator r of block cb belongs to centroid cb*32 + 8*(r/4) + 4*half + r%4 and point t.
    float m1 = __builtin_inff(), m2 = __builtin_inff();   // m1 <= m2
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const float4 c4 = *reinterpret_cast<const float4*>(cnorm + cb * 32 + 8 * q + 4 * half);
            const float cn[4] = {c4.x, c4.y, c4.z, c4.w};
#pragma unroll
            for (int m = 0; m < 4; m++) {
                const float sc = fmaf(-2.f, acc[cb][4 * q + m], cn[m]);   // +inf beyond centroid_num
                m2 = __builtin_amdgcn_fmed3f(m1, m2, sc);   // the second smallest of the three
                m1 = fminf(m1, sc);
            }
        }
    }
    {
        const float o1 = lane_xor<32>(m1), o2 = lane_xor<32>(m2);   // the other half of the point's centroids
        m2 = fminf(fmaxf(m1, o1), fminf(m2, o2));
        m1 = fminf(m1, o1);
    }
    // ---- second sweep: the centroids within the band of the second smallest score
    const float limit = fminf(m2 + assign_band(a.dim, x_norm[t], max_cn), FLT_MAX);   // one centroid only: every valid score passes
    uint32_t found = 0;
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const float4 c4 = *reinterpret_cast<const float4*>(cnorm + cb * 32 + 8 * q + 4 * half);
            const bool h0 = fmaf(-2.f, acc[cb][4 * q], c4.x) <= limit, h1 = fmaf(-2.f, acc[cb][4 * q + 1], c4.y) <= limit,
                       h2 = fmaf(-2.f, acc[cb][4 * q + 2], c4.z) <= limit, h3 = fmaf(-2.f, acc[cb][4 * q + 3], c4.w) <= limit;
            if (h0 | h1 | h2 | h3) {
                const uint32_t c_first = cb * 32 + 8 * q + 4 * half;
                const bool h[4] = {h0, h1, h2, h3};
#pragma unroll
                for (int m = 0; m < 4; m++) {
                    if (h[m]) {
                        if (found < kKeep) cand_by_lane[lane * kKeep + found] = c_first + m;
                        found++;
                    }
                }
            }
        }
    }
    const bool crowded = found > kKeep;
    const uint32_t mine = crowded ? kKeep : found;
    uint32_t pair_count;
    const uint32_t first = wave_exclusive_scan(mine, pair_count);
    lane_first[lane] = first;
    lane_pairs[lane] = mine;
    for (uint32_t k = 0; k < mine; k++) pairs[first + k] = (static_cast<uint32_t>(t) << 16) | cand_by_lane[lane * kKeep + k];
    __builtin_amdgcn_wave_barrier();

    // ---- exact distances of the pairs: one pair per group of 8 lanes, kExactSteps steps in flight.  With eight blocks
    // that is 96 pairs, more than a wavefront usually has, so the pass costs dim / 32 memory round trips and not three
    // times that: the 128 accumulators are dead by now and their registers hold the rows on their way in.  With fewer
    // blocks the registers are worth more as a further wavefront per SIMD.
    constexpr int kExactSteps = CB >= 8 ? 12 : 4;
    const int g = lane >> 3, t8 = lane & 7;
    const uint32_t last = a.num - 1;
    for (uint32_t s0 = 0; s0 < pair_count; s0 += 8 * kExactSteps) {
        const float* xr[kExactSteps];
        const float* cr[kExactSteps];
        float part[kExactSteps];
#pragma unroll
        for (int u = 0; u < kExactSteps; u++) {
            const uint32_t pair = s0 + u * 8 + g;
            const uint32_t pc = pairs[pair < pair_count ? pair : 0u];
            const uint32_t pt = wave_base + (pc >> 16);
            xr[u] = a.data + static_cast<size_t>(pt < a.num ? pt : last) * a.dim;
            cr[u] = a.centroids + static_cast<size_t>(pc & 0xffffu) * a.dim;
            part[u] = 0.f;
        }
        for (uint32_t d0 = t8 * 4; d0 < a.dim; d0 += 32) {
            float4 xv[kExactSteps], cv[kExactSteps];
#pragma unroll
            for (int u = 0; u < kExactSteps; u++) {
                xv[u] = *reinterpret_cast<const float4*>(xr[u] + d0);
                cv[u] = *reinterpret_cast<const float4*>(cr[u] + d0);
            }
#pragma unroll
            for (int u = 0; u < kExactSteps; u++) part[u] = sqdist4(xv[u], cv[u], part[u]);
        }
#pragma unroll
        for (int u = 0; u < kExactSteps; u++) {
            const uint32_t pair = s0 + u * 8 + g;
            const float sq = row_sum<1>(part[u]);   // 8-lane groups
            if (t8 == 0 && pair < pair_count) exact[pair] = finish_distance(sq, a.metric);
        }
    }
    __builtin_amdgcn_wave_barrier();
    // smallest two by (distance, centroid id); lane i < 32 owns point i and reads the pairs of both its halves
    float d0 = FLT_MAX, d1 = FLT_MAX;
    uint32_t c0 = kInvalid, c1 = kInvalid;
#pragma unroll
    for (int hh = 0; hh < 2; hh++) {
        const uint32_t from = lane_first[t + 32 * hh], n = lane_pairs[t + 32 * hh];
#pragma unroll
        for (uint32_t k = 0; k < kKeep; k++)
            if (k < n) nearest_two(exact[from + k], pairs[from + k] & 0xffffu, d0, c0, d1, c1);
    }
    // A point with more than kKeep centroids within the band in one half (near-coincident centroids): every centroid
    // is measured, eight at a time by the same groups of 8 lanes, and the groups' nearest two are combined.
    uint64_t crowded_points = ballot(crowded);
    crowded_points = (crowded_points | (crowded_points >> 32)) & 0xffffffffull;
    while (crowded_points) {
        const int fp = __ffsll(static_cast<long long>(crowded_points)) - 1;
        crowded_points &= crowded_points - 1;
        const uint32_t pt = wave_base + fp;
        const float* xrow = a.data + static_cast<size_t>(pt < a.num ? pt : last) * a.dim;
        float bd0 = FLT_MAX, bd1 = FLT_MAX;
        uint32_t bc0 = kInvalid, bc1 = kInvalid;
        for (uint32_t cbase = 0; cbase < a.centroid_num; cbase += 8) {
            const uint32_t cid = cbase + g;
            const float* crow = a.centroids + static_cast<size_t>(cid < a.centroid_num ? cid : 0u) * a.dim;
            float part = 0.f;
            for (uint32_t dd = t8 * 4; dd < a.dim; dd += 32)
                part = sqdist4(*reinterpret_cast<const float4*>(xrow + dd), *reinterpret_cast<const float4*>(crow + dd), part);
            const float sq = row_sum<1>(part);
            if (cid < a.centroid_num) nearest_two(finish_distance(sq, a.metric), cid, bd0, bc0, bd1, bc1);
        }
#pragma unroll
        for (int m = 8; m <= 32; m <<= 1) {   // the eight groups hold disjoint sets of centroids
            const float od0 = __shfl_xor(bd0, m), od1 = __shfl_xor(bd1, m);
            const uint32_t oc0 = __shfl_xor(bc0, m), oc1 = __shfl_xor(bc1, m);
            nearest_two(od0, oc0, bd0, bc0, bd1, bc1);
            nearest_two(od1, oc1, bd0, bc0, bd1, bc1);
        }
        if (lane == fp) {
            d0 = bd0; c0 = bc0;
            d1 = bd1; c1 = bc1;
        }
    }
    (void) c1;

    const uint32_t p = wave_base + lane;
    if (lane < 32 && p < a.num) {
        // reference partition_kernel.cuh:55-64: boundary iff a second centroid exists and d(2)/d(1) <= factor
        const bool boundary = a.centroid_num > 1 && (d1 / d0 <= a.boundary_factor);
        a.segment_indexes[static_cast<size_t>(p) * 3] = c0;
        a.segment_indexes[static_cast<size_t>(p) * 3 + 2] = boundary ? 0u : kInvalid;
        if (a.nearest_dists) {
            a.nearest_dists[static_cast<size_t>(p) * 2] = d0;
            a.nearest_dists[static_cast<size_t>(p) * 2 + 1] = d1;
        }
        atomicAdd(&hist[c0], 1u);
        if (boundary) atomicAdd(&hist[a.centroid_num], 1u);
    }
    __syncthreads();
    for (uint32_t i = threadIdx.x; i <= a.centroid_num; i += 256)
        a.tile_hist[static_cast<size_t>(i) * gridDim.x + blockIdx.x] = hist[i];
}

// Assignment for at most 32 centroids of at most 128 dims, the shape that is bound by reading the points once.
// NQ = number of 32-dim chunks per row.  The whole centroid matrix sits in LDS for the life of the workgroup, so
// after the one barrier that publishes it the four wavefronts run without meeting again.  Each wavefront issues
// the loads of all its 32 points at once (coalesced, 16 KB in flight at 128 dims), passes them chunk by chunk
// through a private LDS tile into the matrix-instruction operand layout and KEEPS those operand registers, so the
// exact pass over the centroids the ranking leaves reads no point a second time: lane (i, half) rescans its half of
// row i against centroid rows in LDS and the two halves are added.
template <int NQ>
__global__ __launch_bounds__(256) void assign_resident_kernel(AssignArgs a) {
    extern __shared__ __align__(16) float smem[];
    constexpr int DP = 32 * NQ;           // padded dims
    constexpr int CS = DP + 4;            // centroid row stride
    float* cent = smem;                                            // [32][CS], zero outside centroid_num x dim
    float* x_tile = cent + 32 * CS;                                // [4 waves][32][kLdsStride]
    float* cnorm = x_tile + 4 * 32 * kLdsStride;                   // [32]: ||c||^2, +inf beyond centroid_num
    uint32_t* hist = reinterpret_cast<uint32_t*>(cnorm + 32);      // [C + 1]

    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int half = lane >> 5, t = lane & 31;
    const uint32_t wave_base = blockIdx.x * kTilePoints + wave * 32;
    float* xw = x_tile + wave * 32 * kLdsStride;

    float4 xpre[NQ][4];   // chunk c: 8 lanes x float4 per row, 8 rows per step
#pragma unroll
    for (int c = 0; c < NQ; c++)
#pragma unroll
        for (int it = 0; it < 4; it++) {
            const uint32_t p = wave_base + it * 8 + (lane >> 3), d0 = c * 32 + (lane & 7) * 4;
            xpre[c][it] = (p < a.num && d0 < a.dim) ? *reinterpret_cast<const float4*>(a.data + static_cast<size_t>(p) * a.dim + d0)
                                                    : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    for (uint32_t idx = threadIdx.x; idx < 32 * (DP / 4); idx += 256) {
        const uint32_t row = idx / (DP / 4), d0 = (idx % (DP / 4)) * 4;
        *reinterpret_cast<float4*>(cent + row * CS + d0) =
            (row < a.centroid_num && d0 < a.dim) ? *reinterpret_cast<const float4*>(a.centroids + static_cast<size_t>(row) * a.dim + d0)
                                                 : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    for (uint32_t i = threadIdx.x; i <= a.centroid_num; i += 256) hist[i] = 0;
    if (threadIdx.x < 32) cnorm[threadIdx.x] = threadIdx.x < a.centroid_num ? a.centroid_norms[threadIdx.x] : __builtin_inff();
    __syncthreads();

    float16v acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f;
    float4 xr[NQ][4];   // this lane's operand share of row t: dims c*32 + q*8 + 4*half .. +3
#pragma unroll
    for (int c = 0; c < NQ; c++) {
#pragma unroll
        for (int it = 0; it < 4; it++)
            *reinterpret_cast<float4*>(xw + (it * 8 + (lane >> 3)) * kLdsStride + (lane & 7) * 4) = xpre[c][it];
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int q = 0; q < 4; q++) {
            xr[c][q] = *reinterpret_cast<const float4*>(xw + t * kLdsStride + q * 8 + 4 * half);
            const float4 bv = *reinterpret_cast<const float4*>(cent + t * CS + c * 32 + q * 8 + 4 * half);
            // centroids as the A operand, points as B: lane (t, half) ends with the scores of point t
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(bv.x, xr[c][q].x, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(bv.y, xr[c][q].y, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(bv.z, xr[c][q].z, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(bv.w, xr[c][q].w, acc, 0, 0, 0);
        }
        __builtin_amdgcn_wave_barrier();
    }

    // ---- ranking in registers (see assign_band): accumulator r belongs to centroid 8*(r/4) + 4*half + r%4 and point t.
    // The two smallest scores of the point, then the centroids within the band of the second smallest as a bit mask
    // (bit = centroid id) that both lanes of the point share.
    float xsq = 0.f;
#pragma unroll
    for (int c = 0; c < NQ; c++)
#pragma unroll
        for (int q = 0; q < 4; q++)
            xsq = fmaf(xr[c][q].x, xr[c][q].x, fmaf(xr[c][q].y, xr[c][q].y, fmaf(xr[c][q].z, xr[c][q].z, fmaf(xr[c][q].w, xr[c][q].w, xsq))));
    xsq += lane_xor<32>(xsq);
    float max_cn = t < static_cast<int>(a.centroid_num) ? cnorm[t] : 0.f;
#pragma unroll
    for (int m = 16; m >= 1; m >>= 1) max_cn = fmaxf(max_cn, __shfl_xor(max_cn, m));
    float sc[16];
    float m1 = __builtin_inff(), m2 = __builtin_inff();   // m1 <= m2
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const float4 c4 = *reinterpret_cast<const float4*>(cnorm + 8 * q + 4 * half);
        const float cn[4] = {c4.x, c4.y, c4.z, c4.w};
#pragma unroll
        for (int m = 0; m < 4; m++) {
            sc[4 * q + m] = fmaf(-2.f, acc[4 * q + m], cn[m]);   // +inf beyond centroid_num
            m2 = __builtin_amdgcn_fmed3f(m1, m2, sc[4 * q + m]);
            m1 = fminf(m1, sc[4 * q + m]);
        }
    }
    {
        const float o1 = lane_xor<32>(m1), o2 = lane_xor<32>(m2);
        m2 = fminf(fmaxf(m1, o1), fminf(m2, o2));
        m1 = fminf(m1, o1);
    }
    const float limit = fminf(m2 + assign_band(a.dim, xsq, max_cn), FLT_MAX);   // one centroid only: every valid score passes
    uint32_t within = 0;
#pragma unroll
    for (int r = 0; r < 16; r++)
        if (sc[r] <= limit) within |= 1u << (8 * (r / 4) + (r % 4));
    within <<= 4 * half;
    within |= lane_xor<32>(within);

    // exact distances of those centroids from the kept registers, lowest id first; smallest two by (distance, centroid id)
    float d0 = FLT_MAX, d1 = FLT_MAX;
    uint32_t c0 = kInvalid, c1 = kInvalid;
    while (ballot(within != 0)) {
        const bool have = within != 0;
        const uint32_t ck = have ? static_cast<uint32_t>(__ffs(static_cast<int>(within))) - 1u : 0u;
        within &= within - 1;
        const float* crow = cent + ck * CS + 4 * half;
        float part = 0.f;
#pragma unroll
        for (int c = 0; c < NQ; c++)
#pragma unroll
            for (int q = 0; q < 4; q++) part = sqdist4(xr[c][q], *reinterpret_cast<const float4*>(crow + c * 32 + q * 8), part);
        const float sq = part + lane_xor<32>(part);
        if (have) nearest_two(finish_distance(sq, a.metric), ck, d0, c0, d1, c1);
    }
    (void) c1;

    const uint32_t p = wave_base + lane;
    if (lane < 32 && p < a.num) {
        // reference partition_kernel.cuh:55-64: boundary iff a second centroid exists and d(2)/d(1) <= factor
        const bool boundary = a.centroid_num > 1 && (d1 / d0 <= a.boundary_factor);
        a.segment_indexes[static_cast<size_t>(p) * 3] = c0;
        a.segment_indexes[static_cast<size_t>(p) * 3 + 2] = boundary ? 0u : kInvalid;
        if (a.nearest_dists) {
            a.nearest_dists[static_cast<size_t>(p) * 2] = d0;
            a.nearest_dists[static_cast<size_t>(p) * 2 + 1] = d1;
        }
        atomicAdd(&hist[c0], 1u);
        if (boundary) atomicAdd(&hist[a.centroid_num], 1u);
    }
    __syncthreads();
    for (uint32_t i = threadIdx.x; i <= a.centroid_num; i += 256)
        a.tile_hist[static_cast<size_t>(i) * gridDim.x + blockIdx.x] = hist[i];
}

size_t assign_resident_lds_bytes(int nq, uint32_t centroid_num) {
    return (static_cast<size_t>(32) * (32 * nq + 4) + 4 * 32 * kLdsStride + 32) * sizeof(float) + (centroid_num + 1) * sizeof(uint32_t);
}

// exclusive scan over tiles, one workgroup per bin; also emits the bin totals (segment lengths)
constexpr int kScanThreads = 1024;
__global__ __launch_bounds__(kScanThreads) void tile_scan_kernel(uint32_t* tile_hist, uint32_t tiles, uint32_t* totals) {
    __shared__ uint32_t wave_total[kScanThreads / 64];
    const uint32_t bin = blockIdx.x;
    const int lane = lane_id(), wave = threadIdx.x >> 6;
    const uint32_t per = ceil_div(tiles, static_cast<uint32_t>(kScanThreads));
    const uint32_t begin = min(threadIdx.x * per, tiles), end = min(begin + per, tiles);
    uint32_t sum = 0;
    uint32_t* const row = tile_hist + static_cast<size_t>(bin) * tiles;
    for (uint32_t i = begin; i < end; i++) sum += row[i];
    uint32_t inclusive = sum;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint32_t below = static_cast<uint32_t>(__shfl_up(static_cast<int>(inclusive), d));
        if (lane >= d) inclusive += below;
    }
    if (lane == 63) wave_total[wave] = inclusive;
    __syncthreads();
    uint32_t before = 0, total = 0;
#pragma unroll
    for (int w = 0; w < kScanThreads / 64; w++) {
        const uint32_t v = wave_total[w];
        before += w < wave ? v : 0u;
        total += v;
    }
    if (threadIdx.x == 0) totals[bin] = total;
    uint32_t run = before + inclusive - sum;
    for (uint32_t i = begin; i < end; i++) {
        const uint32_t v = row[i];
        row[i] = run;
        run += v;
    }
}

// slot = number of earlier points (in point order) of the same segment; same for the boundary list
__global__ __launch_bounds__(kTilePoints) void slot_kernel(uint32_t* segment_indexes, const uint32_t* tile_base_counts, uint32_t num,
                                                           uint32_t centroid_num) {
    __shared__ uint32_t seg[kTilePoints];
    __shared__ uint32_t bnd[kTilePoints];
    const uint32_t p = blockIdx.x * kTilePoints + threadIdx.x;
    const bool live = p < num;
    const uint32_t my_seg = live ? segment_indexes[static_cast<size_t>(p) * 3] : kInvalid;
    const uint32_t my_b = live ? segment_indexes[static_cast<size_t>(p) * 3 + 2] : kInvalid;
    seg[threadIdx.x] = my_seg;
    bnd[threadIdx.x] = my_b;
    __syncthreads();
    if (!live) return;
    uint32_t rank = 0, brank = 0;
    for (uint32_t j = 0; j < threadIdx.x; j++) {
        rank += seg[j] == my_seg;
        brank += bnd[j] != kInvalid;
    }
    const uint32_t* base = tile_base_counts + blockIdx.x;   // bin-major: bin b of this tile is base[b * tiles]
    segment_indexes[static_cast<size_t>(p) * 3 + 1] = base[static_cast<size_t>(my_seg) * gridDim.x] + rank;
    if (my_b != kInvalid) segment_indexes[static_cast<size_t>(p) * 3 + 2] = base[static_cast<size_t>(centroid_num) * gridDim.x] + brank;
}

// reorder_kernel (partition_kernel.cuh:68-100).  One wavefront moves kReorderRows consecutive points: their source
// rows are one contiguous piece of memory, read as a flat run of float4 with every lane busy whatever the dimension
// (several loads in flight per lane); lanes 0..rows-1 hold the destination rows, fetched per element by a lane read.
constexpr uint32_t kReorderRows = 8;
__global__ __launch_bounds__(256) void reorder_kernel(const float* data, float* reorder_data, const uint32_t* segment_indexes,
                                                      uint32_t* map, const uint32_t* segment_starts, uint32_t num, uint32_t dim,
                                                      uint32_t point_id_offset) {
    const int lane = lane_id();
    const uint32_t first = (blockIdx.x * 4 + (threadIdx.x >> 6)) * kReorderRows;
    if (first >= num) return;
    const uint32_t rows = min(kReorderRows, num - first);
    uint32_t rid = 0, brow = kInvalid;
    if (static_cast<uint32_t>(lane) < rows) {
        const uint32_t* si = segment_indexes + static_cast<size_t>(first + lane) * 3;
        rid = segment_starts[si[0]] + si[1];
        if (si[2] != kInvalid) brow = num + si[2];
        map[rid] = first + lane + point_id_offset;
        if (brow != kInvalid) map[brow] = first + lane + point_id_offset;
    }
    const uint32_t q = dim / 4, total = rows * q;
    const float4* src = reinterpret_cast<const float4*>(data + static_cast<size_t>(first) * dim);
    float4* out = reinterpret_cast<float4*>(reorder_data);
    for (uint32_t e0 = 0; e0 < total; e0 += 256) {
        float4 v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const uint32_t e = e0 + u * 64 + lane;
            if (e < total) v[u] = src[e];
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const uint32_t e = e0 + u * 64 + lane;
            const uint32_t row = min(e / q, rows - 1), col = e - row * q;
            const uint32_t r = __shfl(rid, static_cast<int>(row)), b = __shfl(brow, static_cast<int>(row));
            if (e < total) {
                out[static_cast<size_t>(r) * q + col] = v[u];
                if (b != kInvalid) out[static_cast<size_t>(b) * q + col] = v[u];
            }
        }
    }
}

// sample_kernel (partition_kernel.cuh:7-20)
__global__ __launch_bounds__(256) void sample_rows_kernel(const float* data, float* sample, const uint32_t* ids, uint32_t count, uint32_t dim) {
    const int lane = lane_id();
    const uint32_t i = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (i >= count) return;
    const float* src = data + static_cast<size_t>(ids[i]) * dim;
    float* dst = sample + static_cast<size_t>(i) * dim;
    for (uint32_t d0 = lane * 4; d0 < dim; d0 += 256) *reinterpret_cast<float4*>(dst + d0) = *reinterpret_cast<const float4*>(src + d0);
}

__global__ __launch_bounds__(256) void row_norms_kernel(const float* rows, uint32_t count, uint32_t dim, float* norms) {
    const int lane = lane_id();
    const uint32_t i = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (i >= count) return;
    float acc = 0.f;
    for (uint32_t d = lane; d < dim; d += 64) {
        const float v = rows[static_cast<size_t>(i) * dim + d];
        acc = fmaf(v, v, acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) norms[i] = acc;
}

// ---- greedy k-means++ seeding (cuvs::cluster::kmeans::fit initialises with its k-means++ family by default) ----
// Step s draws 2 + floor(ln k) candidate rows with probability min_dist[i] / sum (uniformly for s = 0) and keeps the
// one that leaves the smallest potential sum_i min(min_dist[i], |x_i - candidate|^2); the distance kernel then lowers
// min_dist with the distances to the winner.  Draw j of step s is a counter-based hash of (seed, 16 s + j), so a run
// is reproducible and a CPU restatement can follow it.
constexpr uint32_t kSeedTrials = 8;        // most candidates per step
constexpr uint32_t kSeedPoints = 64;       // sample rows per workgroup of the trial kernel

__host__ __device__ inline uint32_t seed_trials(uint32_t k) {
    uint32_t t = 2;
    for (uint32_t v = k; v >= 3; v = static_cast<uint32_t>(v / 2.718281828459045)) t++;
    return t > kSeedTrials ? kSeedTrials : t;
}
__device__ __forceinline__ uint32_t seed_hash(uint32_t seed, uint32_t step) {
    uint32_t x = seed * 0x9E3779B9u + step * 0x85EBCA6Bu + 0x6A09E667u;
    x ^= x >> 16; x *= 0x7FEB352Du; x ^= x >> 15; x *= 0x846CA68Bu; x ^= x >> 16;
    return x;
}
__device__ __forceinline__ double shfl_up_f64(double v, int delta) { return __shfl_up(v, delta); }
__device__ __forceinline__ double shfl_f64(double v, int src) { return __shfl(v, src); }

// One wavefront: first index i in [0, len) with load(i) > 0 whose running sum (entries 0..i) exceeds target, and the
// sum of the entries before it; the last positive entry if no running sum gets there (rounding at the upper end).
template <class Load>
__device__ __forceinline__ uint32_t wave_locate(Load load, uint32_t len, double target, double& before, int lane) {
    const uint32_t seg = (len + 63) / 64;
    const uint32_t lo = lane * seg < len ? lane * seg : len, hi = lo + seg < len ? lo + seg : len;
    double local = 0.0;
    for (uint32_t i = lo; i < hi; i++) local += load(i);
    double incl = local;
    for (int off = 1; off < 64; off <<= 1) {
        const double t = shfl_up_f64(incl, off);
        if (lane >= off) incl += t;
    }
    double run = incl - local;
    uint32_t found = 0xffffffffu, last = 0xffffffffu;
    double run_found = 0.0, run_last = 0.0;
    for (uint32_t i = lo; i < hi; i++) {
        const double v = load(i);
        if (v > 0.0) {
            last = i;
            run_last = run;
            if (found == 0xffffffffu && run + v > target) { found = i; run_found = run; }
        }
        run += v;
    }
    const uint64_t hit = ballot(found != 0xffffffffu);
    if (hit) {
        const int src = __builtin_ctzll(hit);
        before = shfl_f64(run_found, src);
        return static_cast<uint32_t>(__shfl(static_cast<int>(found), src));
    }
    const uint64_t any = ballot(last != 0xffffffffu);
    if (!any) { before = 0.0; return 0; }
    const int src = 63 - __builtin_clzll(any);
    before = shfl_f64(run_last, src);
    return static_cast<uint32_t>(__shfl(static_cast<int>(last), src));
}

// one workgroup of 16 wavefronts: chunk sums of min_dist, then wavefront j draws candidate j
__global__ __launch_bounds__(1024) void kmeanspp_pick_kernel(uint32_t n, const float* min_dist, uint32_t seed, uint32_t step, uint32_t trials,
                                                            uint32_t* candidates) {
    __shared__ double part[1024];
    const uint32_t t = threadIdx.x;
    const int lane = lane_id();
    const uint32_t wave = t >> 6;
    if (step == 0) {
        if (t < trials) candidates[t] = seed_hash(seed, 0) % n;
        return;
    }
    const uint32_t chunk = (n + 1023) / 1024;
    {
        const uint32_t lo = t * chunk < n ? t * chunk : n, hi = lo + chunk < n ? lo + chunk : n;
        double acc = 0.0;
        for (uint32_t i = lo; i < hi; i++) acc += static_cast<double>(min_dist[i]);
        part[t] = acc;
    }
    __syncthreads();
    if (wave >= trials) return;
    double total = 0.0;
    for (uint32_t i = lane * 16; i < lane * 16 + 16; i++) total += part[i];
    for (int off = 32; off >= 1; off >>= 1) total += __shfl_xor(total, off);
    uint32_t cand = seed_hash(seed, 16 * step) % n;      // every row already coincides with a centroid
    if (total > 0.0) {
        const uint32_t h = seed_hash(seed, 16 * step + wave);
        const double target = static_cast<double>(h >> 8) * (1.0 / 16777216.0) * total;
        double before = 0.0, unused = 0.0;
        const double* pp = part;
        const uint32_t c = wave_locate([pp](uint32_t i) { return pp[i]; }, 1024, target, before, lane);
        const uint32_t base = c * chunk, len = (base + chunk < n ? base + chunk : n) - base;
        const float* md = min_dist + base;
        cand = base + wave_locate([md](uint32_t i) { return static_cast<double>(md[i]); }, len, target - before, unused, lane);
    }
    if (lane == 0) candidates[wave] = cand;
}

// 64 sample rows per workgroup, 16 per wavefront: potential of every candidate over these rows, in double
__global__ __launch_bounds__(256) void kmeanspp_trial_kernel(const float* sample, uint32_t n, uint32_t dim, const float* min_dist,
                                                             const uint32_t* candidates, uint32_t trials, double* partial) {
    __shared__ double wave_pot[4][kSeedTrials];
    const int lane = lane_id();
    const uint32_t wave = threadIdx.x >> 6;
    double pot[kSeedTrials];
#pragma unroll
    for (uint32_t j = 0; j < kSeedTrials; j++) pot[j] = 0.0;
    for (uint32_t r = 0; r < kSeedPoints / 4; r++) {
        const uint32_t i = blockIdx.x * kSeedPoints + wave * (kSeedPoints / 4) + r;
        if (i >= n) break;
        const float* x = sample + static_cast<size_t>(i) * dim;
        const float md = min_dist[i];
#pragma unroll
        for (uint32_t j = 0; j < kSeedTrials; j++) {
            if (j >= trials) break;
            const float* c = sample + static_cast<size_t>(candidates[j]) * dim;
            float acc = 0.f;
            for (uint32_t d0 = lane * 4; d0 < dim; d0 += 256) {
                const float4 a = *reinterpret_cast<const float4*>(x + d0);
                const float4 b = *reinterpret_cast<const float4*>(c + d0);
                const float dx = a.x - b.x, dy = a.y - b.y, dz = a.z - b.z, dw = a.w - b.w;
                acc = fmaf(dx, dx, acc);
                acc = fmaf(dy, dy, acc);
                acc = fmaf(dz, dz, acc);
                acc = fmaf(dw, dw, acc);
            }
            acc = wave_sum(acc);
            pot[j] += static_cast<double>(fminf(md, acc));
        }
    }
    if (lane == 0)
        for (uint32_t j = 0; j < kSeedTrials; j++) wave_pot[wave][j] = pot[j];
    __syncthreads();
    if (threadIdx.x < kSeedTrials)
        partial[static_cast<size_t>(blockIdx.x) * kSeedTrials + threadIdx.x] =
            wave_pot[0][threadIdx.x] + wave_pot[1][threadIdx.x] + wave_pot[2][threadIdx.x] + wave_pot[3][threadIdx.x];
}

// one workgroup: potentials summed over the trial kernel's workgroups, the smallest wins (the first on a tie); its row
// becomes centroid `step`
__global__ __launch_bounds__(256) void kmeanspp_choose_kernel(const float* sample, uint32_t dim, const double* partial, uint32_t blocks,
                                                              const uint32_t* candidates, uint32_t trials, uint32_t step, float* centroids,
                                                              uint32_t* chosen_rows) {
    __shared__ double slice[kSeedTrials][32];
    __shared__ uint32_t winner;
    const uint32_t j = threadIdx.x >> 5, sl = threadIdx.x & 31;
    double acc = 0.0;
    if (step > 0 && j < trials)
        for (uint32_t b = sl; b < blocks; b += 32) acc += partial[static_cast<size_t>(b) * kSeedTrials + j];
    slice[j][sl] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t best = 0;
        double best_pot = 0.0;
        for (uint32_t c = 0; c < (step > 0 ? trials : 1u); c++) {
            double p = 0.0;
            for (uint32_t q = 0; q < 32; q++) p += slice[c][q];
            if (c == 0 || p < best_pot) { best_pot = p; best = c; }
        }
        winner = candidates[best];
        if (chosen_rows) chosen_rows[step] = winner;
    }
    __syncthreads();
    const float* src = sample + static_cast<size_t>(winner) * dim;
    for (uint32_t d = threadIdx.x; d < dim; d += 256) centroids[static_cast<size_t>(step) * dim + d] = src[d];
}

// one wavefront per sample row: min_dist[i] = min(min_dist[i], |x_i - c|^2) (set on the first step)
__global__ __launch_bounds__(256) void kmeanspp_distance_kernel(const float* sample, uint32_t n, uint32_t dim, const float* centroid, float* min_dist,
                                                                int first) {
    const int lane = lane_id();
    const uint32_t i = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (i >= n) return;
    const float* x = sample + static_cast<size_t>(i) * dim;
    float acc = 0.f;
    for (uint32_t d0 = lane * 4; d0 < dim; d0 += 256) {
        const float4 a = *reinterpret_cast<const float4*>(x + d0);
        const float4 b = *reinterpret_cast<const float4*>(centroid + d0);
        const float dx = a.x - b.x, dy = a.y - b.y, dz = a.z - b.z, dw = a.w - b.w;
        acc = fmaf(dx, dx, acc);
        acc = fmaf(dy, dy, acc);
        acc = fmaf(dz, dz, acc);
        acc = fmaf(dw, dw, acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) min_dist[i] = first ? acc : fminf(min_dist[i], acc);
}

// ---- Lloyd k-means on a sample (stand-in for cuvs::cluster::kmeans::fit, reference partition.cuh:48-54) ----
// The sums are kept in 64-bit fixed point: integer addition does not depend on the order in which the atomics
// arrive, so a fit is reproducible bit for bit.  The scale is the largest power of two for which sample_num values of
// the largest magnitude still fit (2^35 for 500 000 rows of 0..255 data: every value exact; on unit-norm data values
// below 2^-19 are rounded to 2^-43).

// largest |value| of the sample, as the bit pattern of a non-negative float (which orders like the unsigned integer)
__global__ __launch_bounds__(256) void kmeans_range_kernel(const float* sample, size_t count, uint32_t* max_bits) {
    uint32_t m = 0;
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < count; i += static_cast<size_t>(gridDim.x) * 256) {
        const uint32_t b = __float_as_uint(sample[i]) & 0x7fffffffu;
        m = b > m ? b : m;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const uint32_t o = static_cast<uint32_t>(__shfl_xor(static_cast<int>(m), off));
        m = o > m ? o : m;
    }
    if (lane_id() == 0 && m) atomicMax(max_bits, m);
}

// scale = 2^e with max|x| * n * 2^e < 2^62
__device__ __forceinline__ float kmeans_scale(uint32_t max_bits, uint32_t n) {
    const float bound = fmaxf(__uint_as_float(max_bits), 1e-30f) * static_cast<float>(n);
    int e = 0;
    frexpf(bound, &e);           // bound < 2^e
    e = 62 - e;
    e = e > 100 ? 100 : e;
    return ldexpf(1.f, e);
}

// one wavefront per sample point: nearest centroid by direct distances, then atomic accumulation
__global__ __launch_bounds__(256) void kmeans_accumulate_kernel(const float* sample, uint32_t n, uint32_t dim, const float* centroids,
                                                                uint32_t k, long long* sums, uint32_t* counts, const uint32_t* max_bits) {
    const int lane = lane_id();
    const int half = lane >> 5, t = lane & 31;
    const uint32_t i = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (i >= n) return;
    const float* x = sample + static_cast<size_t>(i) * dim;
    float best = FLT_MAX;
    uint32_t bc = 0;
    for (uint32_t c0 = 0; c0 < k; c0 += 2) {
        const uint32_t c = c0 + half < k ? c0 + half : c0;
        const float sq = exact_distance_half(x, centroids + static_cast<size_t>(c) * dim, dim, t);
        const float da = read_lane(sq, 0), db = read_lane(sq, 32);
        if (da < best) { best = da; bc = c0; }
        if (c0 + 1 < k && db < best) { best = db; bc = c0 + 1; }
    }
    const float scale = kmeans_scale(*max_bits, n);
    for (uint32_t d = lane; d < dim; d += 64)
        atomicAdd(reinterpret_cast<unsigned long long*>(&sums[static_cast<size_t>(bc) * dim + d]),
                  static_cast<unsigned long long>(__float2ll_rn(x[d] * scale)));   // two's complement: the wrap-around sum is the signed sum
    if (lane == 0) atomicAdd(&counts[bc], 1u);
}

__global__ void kmeans_update_kernel(float* centroids, const long long* sums, const uint32_t* counts, uint32_t k, uint32_t dim, uint32_t n,
                                     const uint32_t* max_bits) {
    const uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= k * dim) return;
    const uint32_t c = idx / dim;
    if (counts[c])   // an empty cluster keeps its centroid
        centroids[idx] = static_cast<float>(static_cast<double>(sums[idx]) / static_cast<double>(kmeans_scale(*max_bits, n)) /
                                            static_cast<double>(counts[c]));
}

size_t assign_lds_bytes(int cb, uint32_t centroid_num) {
    return (static_cast<size_t>(32) * cb * kLdsStride + 4 * 32 * kLdsStride + 32 * cb) * sizeof(float) + (centroid_num + 1) * sizeof(uint32_t);
}

}  // namespace glide

using namespace glide;

namespace {
size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }
}  // namespace

extern "C" {

size_t glide_hip_partition_assign_workspace_bytes(uint32_t num, uint32_t centroid_num) {
    const size_t tiles = ceil_div(num, kTilePoints);
    return tiles * (centroid_num + 1) * 4 + static_cast<size_t>(centroid_num) * 4 + 256;
}

namespace {
// The launches of glide_hip_partition_assign on a checked workspace: norms (centroid_num floats, padded to 256 bytes) followed by the tile histograms.
int assign_on_workspace(const float* data, uint32_t num, uint32_t dim, const float* centroids, uint32_t centroid_num, float boundary_factor,
                        int metric, uint32_t* segment_indexes, uint32_t* segment_lengths, float* nearest_dists, void* workspace, hipStream_t s) {
    const uint32_t tiles = ceil_div(num, kTilePoints);
    float* norms = static_cast<float*>(workspace);
    uint32_t* tile_hist = reinterpret_cast<uint32_t*>(static_cast<unsigned char*>(workspace) + ((static_cast<size_t>(centroid_num) * 4 + 255) / 256) * 256);
    hipLaunchKernelGGL(row_norms_kernel, dim3(ceil_div(centroid_num, 4)), dim3(256), 0, s, centroids, centroid_num, dim, norms);
    AssignArgs a{data, centroids, norms, segment_indexes, tile_hist, nearest_dists, num, dim, centroid_num, boundary_factor, metric};
    const int cb = centroid_num <= 32 ? 1 : centroid_num <= 64 ? 2 : centroid_num <= 128 ? 4 : 8;
    if (centroid_num <= 32 && dim <= 128) {
        const int nq = static_cast<int>(ceil_div(dim, 32u));
        const size_t rlds = assign_resident_lds_bytes(nq, centroid_num);
        switch (nq) {
            case 1: hipLaunchKernelGGL(assign_resident_kernel<1>, dim3(tiles), dim3(256), rlds, s, a); break;
            case 2: hipLaunchKernelGGL(assign_resident_kernel<2>, dim3(tiles), dim3(256), rlds, s, a); break;
            case 3: hipLaunchKernelGGL(assign_resident_kernel<3>, dim3(tiles), dim3(256), rlds, s, a); break;
            default: hipLaunchKernelGGL(assign_resident_kernel<4>, dim3(tiles), dim3(256), rlds, s, a); break;
        }
    } else {
        const size_t lds = assign_lds_bytes(cb, centroid_num);
        if (lds > 64 * 1024) {
            GLIDE_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(&assign_kernel<8>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                              static_cast<int>(lds)));
        }
        switch (cb) {
            case 1: hipLaunchKernelGGL(assign_kernel<1>, dim3(tiles), dim3(256), lds, s, a); break;
            case 2: hipLaunchKernelGGL(assign_kernel<2>, dim3(tiles), dim3(256), lds, s, a); break;
            case 4: hipLaunchKernelGGL(assign_kernel<4>, dim3(tiles), dim3(256), lds, s, a); break;
            default: hipLaunchKernelGGL(assign_kernel<8>, dim3(tiles), dim3(256), lds, s, a); break;
        }
    }
    // every tile has written all centroid_num + 1 bins of its histogram: nothing in the workspace has to start at zero
    hipLaunchKernelGGL(tile_scan_kernel, dim3(centroid_num + 1), dim3(kScanThreads), 0, s, tile_hist, tiles, segment_lengths);
    hipLaunchKernelGGL(slot_kernel, dim3(tiles), dim3(kTilePoints), 0, s, segment_indexes, tile_hist, num, centroid_num);
    return launch_status();
}

int assign_check(const float* data, uint32_t dim, const float* centroids, uint32_t centroid_num, int metric, const uint32_t* segment_indexes,
                 const uint32_t* segment_lengths) {
    if (!data || !centroids || !segment_indexes || !segment_lengths) return GLIDE_ERR_BAD_ARGUMENT;
    if (dim == 0 || centroid_num == 0) return GLIDE_ERR_BAD_ARGUMENT;
    if (metric != GLIDE_METRIC_EUCLIDEAN && metric != GLIDE_METRIC_COSINE) return GLIDE_ERR_BAD_ARGUMENT;
    if (centroid_num > 256 || dim % 4 != 0) return GLIDE_ERR_UNSUPPORTED;   // reference buckets: kernel_config.cuh:224-234
    return GLIDE_OK;
}
}  // namespace

int glide_hip_partition_assign(const float* data, uint32_t num, uint32_t dim, const float* centroids, uint32_t centroid_num,
                               float boundary_factor, int metric, uint32_t* segment_indexes, uint32_t* segment_lengths,
                               float* nearest_dists, void* workspace, size_t workspace_bytes, void* stream) {
    const int rc = assign_check(data, dim, centroids, centroid_num, metric, segment_indexes, segment_lengths);
    if (rc != GLIDE_OK) return rc;
    if (!workspace || workspace_bytes < glide_hip_partition_assign_workspace_bytes(num, centroid_num)) return GLIDE_ERR_BAD_ARGUMENT;
    if (num == 0) return glide_hip_fill_u32(segment_lengths, 0u, centroid_num + 1, stream);
    return assign_on_workspace(data, num, dim, centroids, centroid_num, boundary_factor, metric, segment_indexes, segment_lengths, nearest_dists,
                               workspace, as_stream(stream));
}

// ---- the entry point that allocates nothing ---------------------------------------------------------------------
// glide_hip_partition_assign with its workspace (centroid norms + per-tile histograms) in a file-scope device array,
// for callers that cannot allocate: code under graph capture, serving loops that route batches of new points or
// queries to their partitions.  Every GPU holds its own copy of the array until the process ends; its address on a
// device is looked up once, with that device current, and kept.
constexpr uint32_t kFixedMaxPoints = 65536;   // per call
constexpr size_t kFixedScratchBytes = 1024 + static_cast<size_t>(kFixedMaxPoints / kTilePoints) * (256 + 1) * 4;   // norms | 512 tiles x 257 bins
static __device__ __align__(256) unsigned char scratch[kFixedScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
std::mutex scratch_mutex;
void* scratch_ptr[kMaxDevices];   // device address of `scratch` per device, null until looked up

int scratch_on_current_device(void** out) {
    int device = 0;
    GLIDE_HIP_TRY(hipGetDevice(&device));
    if (device < 0 || device >= kMaxDevices) return GLIDE_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> guard(scratch_mutex);
    if (!scratch_ptr[device]) {
        void* p = nullptr;
        GLIDE_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return GLIDE_ERR_NO_DEVICE;
        scratch_ptr[device] = p;
    }
    *out = scratch_ptr[device];
    return GLIDE_OK;
}
}  // namespace

uint32_t glide_hip_partition_assign_fixed_max_points(void) { return kFixedMaxPoints; }

int glide_hip_partition_assign_fixed(const float* data, uint32_t num, uint32_t dim, const float* centroids, uint32_t centroid_num,
                                     float boundary_factor, int metric, uint32_t* segment_indexes, uint32_t* segment_lengths,
                                     float* nearest_dists, void* stream) {
    int rc = assign_check(data, dim, centroids, centroid_num, metric, segment_indexes, segment_lengths);
    if (rc != GLIDE_OK) return rc;
    if (num > kFixedMaxPoints) return GLIDE_ERR_UNSUPPORTED;   // the array holds the histograms of 65536 points
    static_assert(kFixedScratchBytes >= 1024 + (kFixedMaxPoints / kTilePoints) * 257 * 4, "scratch too small for the largest call");
    void* ws = nullptr;
    if ((rc = scratch_on_current_device(&ws)) != GLIDE_OK) return rc;
    if (num == 0) return glide_hip_fill_u32(segment_lengths, 0u, centroid_num + 1, stream);   // a fill kernel, no memset node
    return assign_on_workspace(data, num, dim, centroids, centroid_num, boundary_factor, metric, segment_indexes, segment_lengths, nearest_dists,
                               ws, as_stream(stream));
}

int glide_hip_reorder_batch(const float* data, uint32_t num, uint32_t dim, const uint32_t* segment_indexes, const uint32_t* segment_starts,
                            uint32_t point_id_offset, float* reorder_data, uint32_t* map, void* stream) {
    if (!data || !segment_indexes || !segment_starts || !reorder_data || !map || dim == 0) return GLIDE_ERR_BAD_ARGUMENT;
    if (dim % 4 != 0) return GLIDE_ERR_UNSUPPORTED;
    if (num == 0) return GLIDE_OK;
    hipLaunchKernelGGL(reorder_kernel, dim3(ceil_div(num, 4 * kReorderRows)), dim3(256), 0, as_stream(stream), data, reorder_data, segment_indexes, map,
                       segment_starts, num, dim, point_id_offset);
    return launch_status();
}

int glide_hip_reorder(const float* data, uint32_t num, uint32_t dim, const uint32_t* segment_indexes, const uint32_t* segment_starts,
                      float* reorder_data, uint32_t* map, void* stream) {
    return glide_hip_reorder_batch(data, num, dim, segment_indexes, segment_starts, 0u, reorder_data, map, stream);
}

int glide_hip_sample_rows(const float* data, uint32_t dim, const uint32_t* sample_ids, uint32_t sample_num, float* sample, void* stream) {
    if (!data || !sample_ids || !sample || dim == 0) return GLIDE_ERR_BAD_ARGUMENT;
    if (dim % 4 != 0) return GLIDE_ERR_UNSUPPORTED;
    if (sample_num == 0) return GLIDE_OK;
    hipLaunchKernelGGL(sample_rows_kernel, dim3(ceil_div(sample_num, 4)), dim3(256), 0, as_stream(stream), data, sample, sample_ids,
                       sample_num, dim);
    return launch_status();
}

size_t glide_hip_kmeans_workspace_bytes(uint32_t cluster_num, uint32_t dim) {
    // sums (i64 per centroid component) | counts (u32 per centroid) | the sample's largest magnitude
    return static_cast<size_t>(cluster_num) * dim * 8 + static_cast<size_t>(cluster_num) * 4 + 256;
}

size_t glide_hip_kmeans_seed_workspace_bytes(uint32_t sample_num) {
    // min_dist (f32 per row) | candidates (8 u32) | per-workgroup potentials of the trial kernel (8 f64 each)
    return align_up(static_cast<size_t>(sample_num) * 4, 256) + 256 + static_cast<size_t>(ceil_div(sample_num, kSeedPoints)) * kSeedTrials * 8;
}

int glide_hip_kmeans_seed(const float* sample, uint32_t sample_num, uint32_t dim, uint32_t cluster_num, uint32_t seed, float* centroids,
                          uint32_t* chosen_rows, void* workspace, size_t workspace_bytes, void* stream) {
    if (!sample || !centroids || !workspace || dim == 0 || cluster_num == 0 || sample_num == 0) return GLIDE_ERR_BAD_ARGUMENT;
    if (dim % 4 != 0) return GLIDE_ERR_UNSUPPORTED;
    if (workspace_bytes < glide_hip_kmeans_seed_workspace_bytes(sample_num) || reinterpret_cast<uintptr_t>(workspace) % 8)
        return GLIDE_ERR_BAD_ARGUMENT;
    if (reinterpret_cast<uintptr_t>(sample) % 16 || reinterpret_cast<uintptr_t>(centroids) % 16) return GLIDE_ERR_BAD_ARGUMENT;
    hipStream_t s = as_stream(stream);
    unsigned char* w = static_cast<unsigned char*>(workspace);
    float* min_dist = reinterpret_cast<float*>(w);
    uint32_t* candidates = reinterpret_cast<uint32_t*>(w + align_up(static_cast<size_t>(sample_num) * 4, 256));
    double* partial = reinterpret_cast<double*>(w + align_up(static_cast<size_t>(sample_num) * 4, 256) + 256);
    const uint32_t trials = seed_trials(cluster_num), blocks = ceil_div(sample_num, kSeedPoints);
    for (uint32_t step = 0; step < cluster_num; step++) {
        hipLaunchKernelGGL(kmeanspp_pick_kernel, dim3(1), dim3(1024), 0, s, sample_num, min_dist, seed, step, trials, candidates);
        if (step > 0)
            hipLaunchKernelGGL(kmeanspp_trial_kernel, dim3(blocks), dim3(256), 0, s, sample, sample_num, dim, min_dist, candidates, trials, partial);
        hipLaunchKernelGGL(kmeanspp_choose_kernel, dim3(1), dim3(256), 0, s, sample, dim, partial, blocks, candidates, trials, step, centroids,
                           chosen_rows);
        if (step + 1 < cluster_num)
            hipLaunchKernelGGL(kmeanspp_distance_kernel, dim3(ceil_div(sample_num, 4)), dim3(256), 0, s, sample, sample_num, dim,
                               centroids + static_cast<size_t>(step) * dim, min_dist, step == 0 ? 1 : 0);
    }
    return launch_status();
}

int glide_hip_kmeans_fit(const float* sample, uint32_t sample_num, uint32_t dim, uint32_t cluster_num, uint32_t iterations,
                         float* centroids, void* workspace, size_t workspace_bytes, void* stream) {
    if (!sample || !centroids || !workspace || dim == 0 || cluster_num == 0 || sample_num == 0) return GLIDE_ERR_BAD_ARGUMENT;
    if (dim % 4 != 0) return GLIDE_ERR_UNSUPPORTED;
    if (workspace_bytes < glide_hip_kmeans_workspace_bytes(cluster_num, dim)) return GLIDE_ERR_BAD_ARGUMENT;
    hipStream_t s = as_stream(stream);
    if (reinterpret_cast<uintptr_t>(workspace) % 8) return GLIDE_ERR_BAD_ARGUMENT;
    long long* sums = static_cast<long long*>(workspace);
    uint32_t* counts = reinterpret_cast<uint32_t*>(sums + static_cast<size_t>(cluster_num) * dim);
    uint32_t* max_bits = counts + cluster_num;
    const size_t words = static_cast<size_t>(cluster_num) * dim * 2 + cluster_num;
    int rc = glide_hip_fill_u32(max_bits, 0u, 1, stream);
    if (rc != GLIDE_OK) return rc;
    const size_t values = static_cast<size_t>(sample_num) * dim;
    hipLaunchKernelGGL(kmeans_range_kernel, dim3(static_cast<uint32_t>(values / 256 < 4096 ? values / 256 + 1 : 4096)), dim3(256), 0, s, sample,
                       values, max_bits);
    for (uint32_t it = 0; it < iterations; it++) {
        rc = glide_hip_fill_u32(reinterpret_cast<uint32_t*>(sums), 0u, words, stream);
        if (rc != GLIDE_OK) return rc;
        hipLaunchKernelGGL(kmeans_accumulate_kernel, dim3(ceil_div(sample_num, 4)), dim3(256), 0, s, sample, sample_num, dim, centroids,
                           cluster_num, sums, counts, max_bits);
        hipLaunchKernelGGL(kmeans_update_kernel, dim3(ceil_div(cluster_num * dim, 256)), dim3(256), 0, s, centroids, sums, counts,
                           cluster_num, dim, sample_num, max_bits);
    }
    return launch_status();
}

}  // extern "C"
