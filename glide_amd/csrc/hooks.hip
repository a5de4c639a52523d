// Test hooks exposing the device primitives one at a time (distance, bitonic network, hash set).
#include "beam.hpp"
#include "host_util.hpp"

namespace glide {

// one 32-lane half per row pair; generic dim (any multiple of 4, looped in 128-dim chunks)
// uint8 rows -> fp32 rows (the reference's large-path kernels cast every byte where they use it, search_kernel.cuh:493-544);
// four values per thread and step, the tail value by value
__global__ __launch_bounds__(256) void widen_u8_kernel(const unsigned char* src, size_t count, float* dst) {
    const size_t quads = count / 4;
    for (size_t q = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; q < quads; q += static_cast<size_t>(gridDim.x) * 256) {
        const uint32_t w = reinterpret_cast<const uint32_t*>(src)[q];
        reinterpret_cast<float4*>(dst)[q] = make_float4(static_cast<float>(w & 0xff), static_cast<float>((w >> 8) & 0xff),
                                                        static_cast<float>((w >> 16) & 0xff), static_cast<float>(w >> 24));
    }
    if (blockIdx.x == 0 && threadIdx.x < count % 4) dst[quads * 4 + threadIdx.x] = static_cast<float>(src[quads * 4 + threadIdx.x]);
}

// Rows of src_dim values into rows of dst_dim values: the first min(src_dim, dst_dim) values of each row, zeros behind
// them.  One thread per destination value, so the stores are coalesced whatever the two row lengths are.
__global__ __launch_bounds__(256) void copy_rows_kernel(const float* src, size_t num, uint32_t src_dim, float* dst, uint32_t dst_dim) {
    const size_t total = num * dst_dim;
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < total; i += static_cast<size_t>(gridDim.x) * 256) {
        const size_t r = i / dst_dim;
        const uint32_t c = static_cast<uint32_t>(i - r * dst_dim);
        dst[i] = c < src_dim ? src[r * src_dim + c] : 0.f;
    }
}

__global__ __launch_bounds__(64) void distance_batch_kernel(const float* a, const float* b, uint32_t n, uint32_t dim,
                                                            int metric, float* out) {
    const int lane = lane_id();
    const int half = lane >> 5, t = lane & 31;
    const uint32_t i = blockIdx.x * 2 + half;
    float acc = 0.f;
    if (i < n) {
        const float* x = a + static_cast<size_t>(i) * dim;
        const float* y = b + static_cast<size_t>(i) * dim;
        for (uint32_t d0 = t * 4; d0 < dim; d0 += 128) {
            acc = sqdist4(*reinterpret_cast<const float4*>(x + d0), *reinterpret_cast<const float4*>(y + d0), acc);
        }
    }
    const float d = finish_distance(half_wave_sum(acc), metric);
    if (i < n && t == 0) out[i] = d;
}

template <int M, bool MERGE_ONLY>
__global__ __launch_bounds__(64) void bitonic_kernel(float* keys, uint32_t* vals, uint32_t batch) {
    constexpr int NR = WaveNet<M>::NR;
    const int lane = lane_id();
    const uint32_t b = blockIdx.x;
    if (b >= batch) return;
    float k[NR];
    uint32_t v[NR];
    const bool live = (M >= 64) || lane < 32;
#pragma unroll
    for (int r = 0; r < NR; r++) {
        const uint32_t e = NR * lane + r;
        k[r] = live ? keys[static_cast<size_t>(b) * M + e] : FLT_MAX;
        v[r] = live ? vals[static_cast<size_t>(b) * M + e] : kInvalid;
    }
    if (MERGE_ONLY) {
        WaveNet<M>::merge(k, v, lane);
    } else {
        WaveNet<M>::sort(k, v, lane);
    }
#pragma unroll
    for (int r = 0; r < NR; r++) {
        const uint32_t e = NR * lane + r;
        if (live) {
            keys[static_cast<size_t>(b) * M + e] = k[r];
            vals[static_cast<size_t>(b) * M + e] = v[r];
        }
    }
}

// keys are inserted strictly one after another (lane 0 only), so flags match a sequential host model; the
// table is staged through LDS to exercise the same ds atomics as the search kernels.
__global__ __launch_bounds__(64) void hashmap_seq_kernel(uint32_t* table, uint32_t bitlen, const uint32_t* keys, uint32_t n,
                                                         uint32_t* flags) {
    extern __shared__ uint32_t lds_table[];
    const int lane = lane_id();
    for (uint32_t i = lane; i < (1u << bitlen); i += 64) lds_table[i] = table[i];
    __syncthreads();
    if (lane == 0)
        for (uint32_t i = 0; i < n; i++) flags[i] = hash_insert(lds_table, bitlen, keys[i]);
    __syncthreads();
    for (uint32_t i = lane; i < (1u << bitlen); i += 64) table[i] = lds_table[i];
}

template <bool MERGE_ONLY>
int launch_bitonic(float* keys, uint32_t* vals, uint32_t m, uint32_t batch, hipStream_t s) {
    switch (m) {
        case 32: hipLaunchKernelGGL((bitonic_kernel<32, MERGE_ONLY>), dim3(batch), dim3(64), 0, s, keys, vals, batch); break;
        case 64: hipLaunchKernelGGL((bitonic_kernel<64, MERGE_ONLY>), dim3(batch), dim3(64), 0, s, keys, vals, batch); break;
        case 128: hipLaunchKernelGGL((bitonic_kernel<128, MERGE_ONLY>), dim3(batch), dim3(64), 0, s, keys, vals, batch); break;
        case 256: hipLaunchKernelGGL((bitonic_kernel<256, MERGE_ONLY>), dim3(batch), dim3(64), 0, s, keys, vals, batch); break;
        case 512: hipLaunchKernelGGL((bitonic_kernel<512, MERGE_ONLY>), dim3(batch), dim3(64), 0, s, keys, vals, batch); break;
        default: return GLIDE_ERR_UNSUPPORTED;
    }
    return launch_status();
}

}  // namespace glide

using namespace glide;

extern "C" {

int glide_hip_distance_batch(const float* a, const float* b, uint32_t n, uint32_t dim, int metric, float* out, void* stream) {
    if (!a || !b || !out || dim == 0) return GLIDE_ERR_BAD_ARGUMENT;
    if (dim % 4 != 0) return GLIDE_ERR_UNSUPPORTED;
    if (n == 0) return GLIDE_OK;
    hipLaunchKernelGGL(distance_batch_kernel, dim3((n + 1) / 2), dim3(64), 0, as_stream(stream), a, b, n, dim, metric, out);
    return launch_status();
}

int glide_hip_widen_u8(const unsigned char* src, size_t count, float* dst, void* stream) {
    if (!src || !dst || reinterpret_cast<uintptr_t>(dst) % 16 || reinterpret_cast<uintptr_t>(src) % 4) return GLIDE_ERR_BAD_ARGUMENT;
    if (count == 0) return GLIDE_OK;
    const size_t quads = (count + 3) / 4;
    const size_t blocks = (quads + 255) / 256;
    hipLaunchKernelGGL(widen_u8_kernel, dim3(static_cast<uint32_t>(blocks < 16384 ? blocks : 16384)), dim3(256), 0, as_stream(stream), src, count, dst);
    return launch_status();
}

int glide_hip_copy_rows(const float* src, uint64_t num, uint32_t src_dim, float* dst, uint32_t dst_dim, void* stream) {
    if (!src || !dst || src_dim == 0 || dst_dim == 0) return GLIDE_ERR_BAD_ARGUMENT;
    if (num == 0) return GLIDE_OK;
    const size_t blocks = (static_cast<size_t>(num) * dst_dim + 255) / 256;
    hipLaunchKernelGGL(copy_rows_kernel, dim3(static_cast<uint32_t>(blocks < 65536 ? blocks : 65536)), dim3(256), 0, as_stream(stream), src,
                       static_cast<size_t>(num), src_dim, dst, dst_dim);
    return launch_status();
}

int glide_hip_bitonic_sort_kv(float* keys, uint32_t* vals, uint32_t m, uint32_t batch, void* stream) {
    if (!keys || !vals) return GLIDE_ERR_BAD_ARGUMENT;
    if (batch == 0) return GLIDE_OK;
    return launch_bitonic<false>(keys, vals, m, batch, as_stream(stream));
}

int glide_hip_bitonic_merge_kv(float* keys, uint32_t* vals, uint32_t m, uint32_t batch, void* stream) {
    if (!keys || !vals) return GLIDE_ERR_BAD_ARGUMENT;
    if (batch == 0) return GLIDE_OK;
    return launch_bitonic<true>(keys, vals, m, batch, as_stream(stream));
}

int glide_hip_hashmap_insert_seq(uint32_t* table, uint32_t bitlen, const uint32_t* keys, uint32_t n, uint32_t* flags, void* stream) {
    if (!table || !keys || !flags) return GLIDE_ERR_BAD_ARGUMENT;
    if (bitlen < 1 || bitlen > 13) return GLIDE_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(hashmap_seq_kernel, dim3(1), dim3(64), (size_t{1} << bitlen) * sizeof(uint32_t), as_stream(stream), table,
                       bitlen, keys, n, flags);
    return launch_status();
}

}  // extern "C"
