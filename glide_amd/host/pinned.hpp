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
