// Measurement yardsticks for the profiles and the benchmark: a plain copy of known size, register-only instruction loops
// and scattered atomics.  Not part of the product library: built into libglide_probes.so, declared in
// include/glide_hip_probes.h, used by bench.py's calibration flags only.
#include "common.hpp"
#include "host_util.hpp"
#include "../../include/glide_hip_probes.h"

namespace glide {

// plain streaming copy of known size: the yardstick that hardware byte counters are scaled with
__global__ __launch_bounds__(256) void copy_kernel(const uint4* src, uint4* dst, size_t n16) {
    size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    for (; i < n16; i += stride) dst[i] = src[i];
}

// Yardstick for the vector-ALU issue rate (no counterpart in the reference): every lane runs `rounds` x 16 independent
// register-only instructions, nothing else.  2048 workgroups of 256 threads keep eight wavefronts on every SIMD.
// MODE 0: fused multiply-add; 1: 32-bit integer add; 2: compare + select (two instructions per step, the pair a
// sorting network is made of); 3: cross-lane move (DPP quad permute) + add.
template <int MODE>
__global__ __launch_bounds__(256) void valu_probe_kernel(uint32_t rounds, float seed, float* out) {
    float v[16];
#pragma unroll
    for (int i = 0; i < 16; i++) v[i] = seed + static_cast<float>(threadIdx.x + i);
    for (uint32_t r = 0; r < rounds; r++) {
#pragma unroll
        for (int i = 0; i < 16; i++) {
            if constexpr (MODE == 0) {
                v[i] = fmaf(v[i], 1.0000001f, 0.5f);
            } else if constexpr (MODE == 1) {
                v[i] = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, v[i]) + 0x9E3779B1u);
            } else if constexpr (MODE == 2) {
                v[i] = v[i] < v[(i + 1) & 15] ? v[(i + 3) & 15] : v[i];
            } else {
                v[i] = __builtin_bit_cast(float, __builtin_bit_cast(int, lane_xor<1>(v[i])) + 1);
            }
        }
    }
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) sum += v[i];
    if (sum == 12345.678f) out[0] = sum;   // keeps the loop alive; practically never taken
}

// The rate of atomic operations on scattered words: every thread issues `rounds` of them on slots of `table` drawn by
// a hash of (thread, round).  MODE 0: 64-bit minimum, nothing returned (what an NN-descent offer is made of); 1: 32-bit
// add whose result is used (what reserves a slot of a reverse list); 2 and 3: as 0, with 2 / 16 adjacent lanes on slots of
// one 128-byte line.
template <int MODE>
__global__ __launch_bounds__(256) void atomic_probe_kernel(unsigned long long* table, uint32_t slot_mask, uint32_t rounds, uint32_t* out) {
    const uint32_t tid = blockIdx.x * 256 + threadIdx.x;
    uint32_t x = tid * 0x9E3779B1u + 0x7F4A7C15u, sum = 0;
    for (uint32_t r = 0; r < rounds; r++) {
        x ^= x << 13;
        x ^= x >> 17;
        x ^= x << 5;
        uint32_t slot = (x * 0x85EBCA6Bu >> 4) & slot_mask;
        if constexpr (MODE >= 2) {   // groups of 2 (MODE 2) or 16 (MODE 3) adjacent lanes share a 128-byte line
            constexpr uint32_t G = MODE == 2 ? 2 : 16;
            const uint32_t leader = static_cast<uint32_t>(__shfl(static_cast<int>(slot), static_cast<int>(threadIdx.x & 63u & ~(G - 1))));
            slot = ((leader & ~15u) | ((leader + (threadIdx.x & (G - 1))) & 15u)) & slot_mask;
        }
        if constexpr (MODE != 1) {
            __hip_atomic_fetch_min(&table[slot], (static_cast<unsigned long long>(x) << 32) | tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
            sum += atomicAdd(reinterpret_cast<uint32_t*>(table) + 2 * slot, 1u);
        }
    }
    if (sum == 0xFFFFFFF1u) out[0] = sum;   // keeps the results alive; practically never taken
}

// The rate at which rows scattered over a table can be read, whatever is done with them: every wavefront walks its own
// pseudo-random sequence of rows and reads each one with 16-byte loads of adjacent lanes, `rows_in_flight` rows requested
// before the first is consumed (ROWS_PER_STEP rows per wave-wide step: a row takes 64 / ROWS_PER_STEP lanes and as many
// loads per lane as its length needs).  This is the memory side of a graph search's scoring loop without its distances,
// its sorting networks and its dependent graph-row fetch.
template <int ROWS_PER_STEP, int STEPS>
__global__ __launch_bounds__(64) void gather_probe_kernel(const float4* table, uint32_t row_count, uint32_t quads_per_row, uint32_t stride_quads,
                                                          uint32_t rows_per_wave, float* out) {
    constexpr int LPR = 64 / ROWS_PER_STEP;
    const int lane = threadIdx.x, g = lane / LPR, t = lane % LPR;
    uint32_t x = (blockIdx.x * 64 + 1) * 0x9E3779B1u + 0x7F4A7C15u;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (uint32_t r = 0; r < rows_per_wave; r += ROWS_PER_STEP * STEPS) {
        uint32_t row[STEPS];
#pragma unroll
        for (int s = 0; s < STEPS; s++) {
            x ^= x << 13;
            x ^= x >> 17;
            x ^= x << 5;
            row[s] = static_cast<uint32_t>((static_cast<unsigned long long>((x + g * 0x85EBCA6Bu) * 0xC2B2AE35u) * row_count) >> 32);
        }
        for (uint32_t c = t; c < quads_per_row; c += LPR) {
            float4 v[STEPS];
#pragma unroll
            for (int s = 0; s < STEPS; s++) v[s] = table[static_cast<size_t>(row[s]) * stride_quads + c];
#pragma unroll
            for (int s = 0; s < STEPS; s++) {
                acc.x += v[s].x;
                acc.y += v[s].y;
                acc.z += v[s].z;
                acc.w += v[s].w;
            }
        }
    }
    if (acc.x + acc.y + acc.z + acc.w == 12345.678f) out[0] = acc.x;   // keeps the loads alive; practically never taken
}

}  // namespace glide

using namespace glide;

extern "C" {

int glide_probe_copy_bytes(void* dst, const void* src, size_t bytes, void* stream) {
    if (!dst || !src || bytes % 16 || reinterpret_cast<uintptr_t>(dst) % 16 || reinterpret_cast<uintptr_t>(src) % 16) return GLIDE_ERR_BAD_ARGUMENT;
    if (bytes == 0) return GLIDE_OK;
    hipLaunchKernelGGL(copy_kernel, dim3(8192), dim3(256), 0, as_stream(stream), static_cast<const uint4*>(src), static_cast<uint4*>(dst), bytes / 16);
    return launch_status();
}

int glide_probe_valu(int mode, uint32_t rounds, float* out, void* stream) {
    if (!out || mode < 0 || mode > 3) return GLIDE_ERR_BAD_ARGUMENT;
    switch (mode) {
        case 0: hipLaunchKernelGGL(valu_probe_kernel<0>, dim3(2048), dim3(256), 0, as_stream(stream), rounds, 1.0f, out); break;
        case 1: hipLaunchKernelGGL(valu_probe_kernel<1>, dim3(2048), dim3(256), 0, as_stream(stream), rounds, 1.0f, out); break;
        case 2: hipLaunchKernelGGL(valu_probe_kernel<2>, dim3(2048), dim3(256), 0, as_stream(stream), rounds, 1.0f, out); break;
        default: hipLaunchKernelGGL(valu_probe_kernel<3>, dim3(2048), dim3(256), 0, as_stream(stream), rounds, 1.0f, out); break;
    }
    return launch_status();
}

int glide_probe_atomic(int mode, unsigned long long* table, uint32_t slots, uint32_t rounds, uint32_t* out, void* stream) {
    if (!table || !out || mode < 0 || mode > 3 || slots < 16 || (slots & (slots - 1)) != 0) return GLIDE_ERR_BAD_ARGUMENT;
    switch (mode) {
        case 0: hipLaunchKernelGGL(atomic_probe_kernel<0>, dim3(2048), dim3(256), 0, as_stream(stream), table, slots - 1, rounds, out); break;
        case 1: hipLaunchKernelGGL(atomic_probe_kernel<1>, dim3(2048), dim3(256), 0, as_stream(stream), table, slots - 1, rounds, out); break;
        case 2: hipLaunchKernelGGL(atomic_probe_kernel<2>, dim3(2048), dim3(256), 0, as_stream(stream), table, slots - 1, rounds, out); break;
        default: hipLaunchKernelGGL(atomic_probe_kernel<3>, dim3(2048), dim3(256), 0, as_stream(stream), table, slots - 1, rounds, out); break;
    }
    return launch_status();
}

int glide_probe_gather(const void* table, uint32_t row_count, uint32_t row_bytes, uint32_t row_stride_bytes, uint32_t waves, uint32_t rows_per_wave, int rows_per_step,
                       float* out, void* stream) {
    if (!table || !out || row_count == 0 || row_bytes == 0 || row_bytes % 16 != 0 || row_stride_bytes % 16 != 0 || row_stride_bytes < row_bytes || waves == 0)
        return GLIDE_ERR_BAD_ARGUMENT;
    const float4* t = static_cast<const float4*>(table);
    const uint32_t quads = row_bytes / 16, stride = row_stride_bytes / 16;
    hipStream_t s = as_stream(stream);
    switch (rows_per_step) {
        case 8: hipLaunchKernelGGL((gather_probe_kernel<8, 2>), dim3(waves), dim3(64), 0, s, t, row_count, quads, stride, rows_per_wave, out); break;
        case 2: hipLaunchKernelGGL((gather_probe_kernel<2, 4>), dim3(waves), dim3(64), 0, s, t, row_count, quads, stride, rows_per_wave, out); break;
        case 1: hipLaunchKernelGGL((gather_probe_kernel<1, 8>), dim3(waves), dim3(64), 0, s, t, row_count, quads, stride, rows_per_wave, out); break;
        default: return GLIDE_ERR_UNSUPPORTED;
    }
    return launch_status();
}

}  // extern "C"
