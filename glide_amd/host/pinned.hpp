// Host arrays in pinned memory: the large path keeps data, kNN graph and graph on the host and stages one partition
// at a time through the GPU (reference GLIDE_large, glide_large.cuh:14-212); pinned memory lets those copies run
// asynchronously next to the kernels.
#pragma once
#include <cstring>
#include <fstream>
#include <iostream>
#include <string>

#include "mdarray.hpp"

namespace glide {

template <typename T>
class pinned_matrix {
public:
    pinned_matrix() = default;
    pinned_matrix(size_t rows, size_t cols) : rows_(rows), cols_(cols) {
        void* p = nullptr;
        hip_try(glide_hip_host_alloc_pinned(&p, rows * cols * sizeof(T)), "glide_hip_host_alloc_pinned");
        ptr_ = static_cast<T*>(p);
    }
    pinned_matrix(pinned_matrix&& o) noexcept : ptr_(o.ptr_), rows_(o.rows_), cols_(o.cols_) { o.ptr_ = nullptr; }
    pinned_matrix& operator=(pinned_matrix&& o) noexcept {
        if (this != &o) { release(); ptr_ = o.ptr_; rows_ = o.rows_; cols_ = o.cols_; o.ptr_ = nullptr; }
        return *this;
    }
    pinned_matrix(const pinned_matrix&) = delete;
    pinned_matrix& operator=(const pinned_matrix&) = delete;
    ~pinned_matrix() { release(); }
    T* data_handle() const { return ptr_; }
    size_t extent(int i) const { return i == 0 ? rows_ : cols_; }
    size_t size() const { return rows_ * cols_; }
    T* row(size_t r) const { return ptr_ + r * cols_; }
private:
    void release() { if (ptr_) glide_hip_host_free_pinned(ptr_); ptr_ = nullptr; }
    T* ptr_ = nullptr;
    size_t rows_ = 0, cols_ = 0;
};

// fbin file straight into pinned memory (load.cuh:8-31 format)
template <typename T>
pinned_matrix<T> load_matrix_pinned(const std::string& path) {
    std::ifstream file(path, std::ios::binary);
    if (!file) std::cerr << "Error opening file: " << path << std::endl;
    uint32_t num = 0, dim = 0;
    file.read(reinterpret_cast<char*>(&num), sizeof(uint32_t));
    file.read(reinterpret_cast<char*>(&dim), sizeof(uint32_t));
    pinned_matrix<T> m(num, dim);
    const size_t chunk = size_t{1} << 28;
    char* dst = reinterpret_cast<char*>(m.data_handle());
    size_t left = m.size() * sizeof(T);
    while (left) {
        const size_t n = left < chunk ? left : chunk;
        file.read(dst, static_cast<std::streamsize>(n));
        dst += n;
        left -= n;
    }
    return m;
}

// A file of points into pinned memory, rows padded by zeros to a multiple of 16 bytes (load.hpp: load_point_data).
template <typename T>
pinned_matrix<T> load_points_pinned(const std::string& path, uint32_t* file_dim = nullptr) {
    std::ifstream file(path, std::ios::binary);
    if (!file) std::cerr << "Error opening file: " << path << std::endl;
    uint32_t num = 0, dim = 0;
    file.read(reinterpret_cast<char*>(&num), sizeof(uint32_t));
    file.read(reinterpret_cast<char*>(&dim), sizeof(uint32_t));
    if (file_dim) *file_dim = dim;
    constexpr uint32_t multiple = 16 / sizeof(T);
    const uint32_t held = (dim + multiple - 1) / multiple * multiple;
    if (held == dim) return load_matrix_pinned<T>(path);
    pinned_matrix<T> m(num, held);
    for (size_t r = 0; r < num; r++) {
        file.read(reinterpret_cast<char*>(m.row(r)), static_cast<std::streamsize>(dim * sizeof(T)));
        std::memset(m.row(r) + dim, 0, (held - dim) * sizeof(T));
    }
    return m;
}

// The first `file_dim` values of every row.
template <typename T>
void save_points_pinned(const std::string& path, const pinned_matrix<T>& m, uint32_t file_dim);

template <typename T>
void save_matrix_pinned(const std::string& path, const pinned_matrix<T>& m) {
    std::ofstream file(path, std::ios::binary);
    uint32_t num = m.extent(0), dim = m.extent(1);
    file.write(reinterpret_cast<const char*>(&num), sizeof(uint32_t));
    file.write(reinterpret_cast<const char*>(&dim), sizeof(uint32_t));
    const size_t chunk = size_t{1} << 28;
    const char* src = reinterpret_cast<const char*>(m.data_handle());
    size_t left = m.size() * sizeof(T);
    while (left) {
        const size_t n = left < chunk ? left : chunk;
        file.write(src, static_cast<std::streamsize>(n));
        src += n;
        left -= n;
    }
}

template <typename T>
void save_points_pinned(const std::string& path, const pinned_matrix<T>& m, uint32_t file_dim) {
    if (file_dim == m.extent(1)) return save_matrix_pinned(path, m);
    std::ofstream file(path, std::ios::binary);
    const uint32_t num = m.extent(0);
    file.write(reinterpret_cast<const char*>(&num), sizeof(uint32_t));
    file.write(reinterpret_cast<const char*>(&file_dim), sizeof(uint32_t));
    for (size_t r = 0; r < m.extent(0); r++) file.write(reinterpret_cast<const char*>(m.row(r)), static_cast<std::streamsize>(file_dim * sizeof(T)));
}

// Size in bytes of one element of an fbin file, from its length: header (num, dim) + num * dim elements.  The reference's
// large executables read uint8 rows (large_preprocess.cu:56); this build also takes fp32 rows in the same layout.
inline size_t fbin_element_bytes(const std::string& path) {
    std::ifstream file(path, std::ios::binary | std::ios::ate);
    if (!file) { std::cerr << "Error opening file: " << path << std::endl; return 0; }
    const size_t bytes = static_cast<size_t>(file.tellg());
    file.seekg(0);
    uint32_t num = 0, dim = 0;
    file.read(reinterpret_cast<char*>(&num), sizeof(uint32_t));
    file.read(reinterpret_cast<char*>(&dim), sizeof(uint32_t));
    const size_t count = static_cast<size_t>(num) * dim;
    return count ? (bytes - 8) / count : 0;
}

// One staging slot for a block of rows: uploaded in their stored type, read by every kernel as fp32.  Float rows are
// copied straight into place; uint8 rows are copied raw (a quarter of the PCIe traffic) and widened on the GPU.
template <typename Data_t>
class staged_rows {
    static_assert(sizeof(Data_t) == 4 || sizeof(Data_t) == 1, "float or uint8 rows");
public:
    staged_rows(size_t max_rows, uint32_t dim) : rows_(max_rows, dim), raw_(sizeof(Data_t) == 1 ? max_rows * dim + 16 : 16) {}
    // on the copy stream
    void upload_async(const Data_t* src, size_t rows, void* stream) {
        hip_try(glide_hip_memcpy_h2d_async(stored(), src, rows * rows_.extent(1) * sizeof(Data_t), stream), "glide_hip_memcpy_h2d_async");
    }
    // on the compute stream, once the copy is known to be complete
    void widen(size_t rows, void* stream) {
        if (sizeof(Data_t) == 1)
            hip_try(glide_hip_widen_u8(static_cast<const unsigned char*>(raw_.get()), rows * rows_.extent(1), rows_.data_handle(), stream),
                    "glide_hip_widen_u8");
    }
    float* data_handle() const { return rows_.data_handle(); }
    // the rows in their stored type (same memory as data_handle() for float rows)
    Data_t* stored() const { return sizeof(Data_t) == 1 ? static_cast<Data_t*>(raw_.get()) : reinterpret_cast<Data_t*>(rows_.data_handle()); }
private:
    device_matrix<float> rows_;
    device_buffer raw_;
};

// two streams + events for "copy partition s+1 while partition s computes"
class stager {
public:
    stager() {
        hip_try(glide_hip_stream_create(&copy_), "glide_hip_stream_create");
        hip_try(glide_hip_stream_create(&compute_), "glide_hip_stream_create");
        for (auto& e : copied_) hip_try(glide_hip_event_create(&e), "glide_hip_event_create");
        for (auto& e : computed_) hip_try(glide_hip_event_create(&e), "glide_hip_event_create");
    }
    ~stager() {
        glide_hip_stream_synchronize(copy_);
        glide_hip_stream_synchronize(compute_);
        for (auto e : copied_) glide_hip_event_destroy(e);
        for (auto e : computed_) glide_hip_event_destroy(e);
        glide_hip_stream_destroy(copy_);
        glide_hip_stream_destroy(compute_);
    }
    void* copy_stream() const { return copy_; }
    void* compute_stream() const { return compute_; }
    // the copy stream may overwrite slot b once the kernels that last used it are done
    void before_copy(int b) { if (used_[b]) hip_try(glide_hip_stream_wait_event(copy_, computed_[b]), "glide_hip_stream_wait_event"); }
    void after_copy(int b) { hip_try(glide_hip_event_record(copied_[b], copy_), "glide_hip_event_record"); }
    void before_compute(int b) { hip_try(glide_hip_stream_wait_event(compute_, copied_[b]), "glide_hip_stream_wait_event"); }
    void after_compute(int b) {
        hip_try(glide_hip_event_record(computed_[b], compute_), "glide_hip_event_record");
        used_[b] = true;
    }
    void sync() {
        hip_try(glide_hip_stream_synchronize(copy_), "glide_hip_stream_synchronize");
        hip_try(glide_hip_stream_synchronize(compute_), "glide_hip_stream_synchronize");
    }
private:
    void* copy_ = nullptr;
    void* compute_ = nullptr;
    void* copied_[2] = {nullptr, nullptr};
    void* computed_[2] = {nullptr, nullptr};
    bool used_[2] = {false, false};
};

}  // namespace glide
