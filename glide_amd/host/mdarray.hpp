// Minimal owning host/device matrices and views with the accessor names the reference code uses on RAFT
// mdarrays (data_handle(), extent(i), size(), operator()), plus the resource handle carrying the stream.
// Device memory, copies and streams all go through the C ABI (include/glide_hip.h); no HIP headers here.
#pragma once
#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "../../include/glide_hip.h"

namespace glide {

struct hip_error : std::runtime_error {   // stands in for raft::cuda_error (RAFT_CUDA_TRY, reference glide_impl.cuh:142)
    int code;
    hip_error(int c, const std::string& what) : std::runtime_error(what + ": " + glide_hip_error_string(c)), code(c) {}
};

inline void hip_try(int code, const char* what) {
    if (code == GLIDE_OK) return;
    if (code == GLIDE_ERR_UNSUPPORTED) throw std::invalid_argument(std::string("Unsupported size in ") + what);  // kernel_config.cuh:48,60
    throw hip_error(code, what);
}

class device_resources {   // reference: raft::device_resources + rmm stream pool (small_build.cu:34-36)
public:
    explicit device_resources(int device = 0) { hip_try(glide_hip_set_device(device), "glide_hip_set_device"); }
    void* stream() const { return nullptr; }   // default stream; every stage is ordered on it
    void sync() const { hip_try(glide_hip_stream_synchronize(nullptr), "glide_hip_stream_synchronize"); }
};

template <typename T, typename I = uint32_t>
struct matrix_view {
    T* ptr = nullptr;
    I rows = 0, cols = 0;
    T* data_handle() const { return ptr; }
    I extent(int i) const { return i == 0 ? rows : cols; }
    size_t size() const { return static_cast<size_t>(rows) * cols; }
    T& operator()(I r, I c) const { return ptr[static_cast<size_t>(r) * cols + c]; }
};
template <typename T, typename I = uint32_t>
struct vector_view {
    T* ptr = nullptr;
    I len = 0;
    T* data_handle() const { return ptr; }
    I extent(int) const { return len; }
    size_t size() const { return len; }
    T& operator()(I i) const { return ptr[i]; }
};
template <typename T, typename I = uint32_t> using host_matrix_view = matrix_view<T, I>;
template <typename T, typename I = uint32_t> using device_matrix_view = matrix_view<T, I>;
template <typename T, typename I = uint32_t> using host_vector_view = vector_view<T, I>;
template <typename T, typename I = uint32_t> using device_vector_view = vector_view<T, I>;

template <typename T, typename I = uint32_t>
class host_matrix {
public:
    host_matrix() = default;
    host_matrix(I rows, I cols) : rows_(rows), cols_(cols), data_(static_cast<size_t>(rows) * cols) {}
    T* data_handle() { return data_.data(); }
    const T* data_handle() const { return data_.data(); }
    I extent(int i) const { return i == 0 ? rows_ : cols_; }
    size_t size() const { return data_.size(); }
    T& operator()(I r, I c) { return data_[static_cast<size_t>(r) * cols_ + c]; }
    host_matrix_view<T, I> view() { return {data_.data(), rows_, cols_}; }
    host_matrix_view<const T, I> view() const { return {data_.data(), rows_, cols_}; }
private:
    I rows_ = 0, cols_ = 0;
    std::vector<T> data_;
};
template <typename T, typename I = uint32_t>
class host_vector {
public:
    host_vector() = default;
    explicit host_vector(I n) : data_(n) {}
    T* data_handle() { return data_.data(); }
    const T* data_handle() const { return data_.data(); }
    I extent(int) const { return static_cast<I>(data_.size()); }
    size_t size() const { return data_.size(); }
    T& operator()(I i) { return data_[i]; }
    host_vector_view<T, I> view() { return {data_.data(), static_cast<I>(data_.size())}; }
    host_vector_view<const T, I> view() const { return {data_.data(), static_cast<I>(data_.size())}; }
private:
    std::vector<T> data_;
};

class device_buffer {   // raw owning allocation
public:
    device_buffer() = default;
    explicit device_buffer(size_t bytes) : bytes_(bytes) { hip_try(glide_hip_malloc(&ptr_, bytes), "glide_hip_malloc"); }
    device_buffer(device_buffer&& o) noexcept : ptr_(o.ptr_), bytes_(o.bytes_) { o.ptr_ = nullptr; o.bytes_ = 0; }
    device_buffer& operator=(device_buffer&& o) noexcept {
        if (this != &o) { release(); ptr_ = o.ptr_; bytes_ = o.bytes_; o.ptr_ = nullptr; o.bytes_ = 0; }
        return *this;
    }
    device_buffer(const device_buffer&) = delete;
    device_buffer& operator=(const device_buffer&) = delete;
    ~device_buffer() { release(); }
    void* get() const { return ptr_; }
    size_t bytes() const { return bytes_; }
private:
    void release() { if (ptr_) glide_hip_free(ptr_); ptr_ = nullptr; }
    void* ptr_ = nullptr;
    size_t bytes_ = 0;
};

template <typename T, typename I = uint32_t>
class device_matrix {
public:
    device_matrix() = default;
    device_matrix(I rows, I cols) : rows_(rows), cols_(cols), buf_(static_cast<size_t>(rows) * cols * sizeof(T)) {}
    T* data_handle() const { return static_cast<T*>(buf_.get()); }
    I extent(int i) const { return i == 0 ? rows_ : cols_; }
    size_t size() const { return static_cast<size_t>(rows_) * cols_; }
    device_matrix_view<T, I> view() const { return {data_handle(), rows_, cols_}; }
private:
    I rows_ = 0, cols_ = 0;
    device_buffer buf_;
};
template <typename T, typename I = uint32_t>
class device_vector {
public:
    device_vector() = default;
    explicit device_vector(I n) : len_(n), buf_(static_cast<size_t>(n) * sizeof(T)) {}
    T* data_handle() const { return static_cast<T*>(buf_.get()); }
    I extent(int) const { return len_; }
    size_t size() const { return len_; }
    device_vector_view<T, I> view() const { return {data_handle(), len_}; }
private:
    I len_ = 0;
    device_buffer buf_;
};

template <typename T>
inline void copy_to_device(T* dst, const T* src, size_t count) {
    hip_try(glide_hip_memcpy_h2d(dst, src, count * sizeof(T), nullptr), "glide_hip_memcpy_h2d");
}
template <typename T>
inline void copy_to_host(T* dst, const T* src, size_t count) {
    hip_try(glide_hip_memcpy_d2h(dst, src, count * sizeof(T), nullptr), "glide_hip_memcpy_d2h");
}

class gpu_timer {   // cudaEvent pairs of the reference (glide_impl.cuh:53-72): seconds between two events
public:
    gpu_timer() {
        hip_try(glide_hip_event_create(&start_), "glide_hip_event_create");
        hip_try(glide_hip_event_create(&stop_), "glide_hip_event_create");
    }
    ~gpu_timer() { glide_hip_event_destroy(start_); glide_hip_event_destroy(stop_); }
    void start() { hip_try(glide_hip_event_record(start_, nullptr), "glide_hip_event_record"); }
    float stop() {
        float ms = 0.f;
        hip_try(glide_hip_event_record(stop_, nullptr), "glide_hip_event_record");
        hip_try(glide_hip_event_elapsed_ms(start_, stop_, &ms), "glide_hip_event_elapsed_ms");
        return ms / 1000.0f;
    }
private:
    void* start_ = nullptr;
    void* stop_ = nullptr;
};

}  // namespace glide
