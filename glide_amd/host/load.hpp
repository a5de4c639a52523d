// File formats of the reference's load.cuh:8-128, byte for byte:
//   matrix (fbin)  u32 num, u32 dim, num*dim values            (.centroid, .reorder, knn file, .graph, data, truth)
//   segment        u32 n, u32 start[n], u32 length[n]          (.segment; n = centroid_num + 1, last = boundary)
//   vector         u32 n, u32 value[n]                         (.map, .sp)
// Files of points (data, queries, .centroid, .reorder) keep whatever row length they have.  In memory their rows are
// held with the length rounded up to a multiple of 16 bytes of the stored type, the added values zero
// (load_point_data / save_point_data): every kernel reads rows in 16-byte pieces, and a zero coordinate changes no
// squared distance, inner product or norm.
#pragma once
#include <fstream>
#include <iostream>
#include <string>

#include "mdarray.hpp"

namespace glide {

template <typename Data_t, typename Index_t = uint32_t>
host_matrix<Data_t, Index_t> load_matrix_data(const std::string& path) {
    std::ifstream file(path, std::ios::binary);
    if (!file) std::cerr << "Error opening file: " << path << std::endl;   // the reference prints and carries on (load.cuh:12-14)
    uint32_t num = 0, dim = 0;
    file.read(reinterpret_cast<char*>(&num), sizeof(uint32_t));
    file.read(reinterpret_cast<char*>(&dim), sizeof(uint32_t));
    host_matrix<Data_t, Index_t> data(num, dim);
    file.read(reinterpret_cast<char*>(data.data_handle()), static_cast<std::streamsize>(data.size() * sizeof(Data_t)));
    return data;
}

inline uint32_t padded_dim(uint32_t dim, uint32_t multiple) { return (dim + multiple - 1) / multiple * multiple; }

// A file of points with its rows padded by zeros to a multiple of `multiple` values (default: 16 bytes' worth of the
// stored type; the .centroid file of uint8 data is float and takes the data's 16).  *file_dim: the row length in the file.
template <typename Data_t, typename Index_t = uint32_t>
host_matrix<Data_t, Index_t> load_point_data(const std::string& path, uint32_t multiple = 16 / sizeof(Data_t), uint32_t* file_dim = nullptr) {
    std::ifstream file(path, std::ios::binary);
    if (!file) std::cerr << "Error opening file: " << path << std::endl;
    uint32_t num = 0, dim = 0;
    file.read(reinterpret_cast<char*>(&num), sizeof(uint32_t));
    file.read(reinterpret_cast<char*>(&dim), sizeof(uint32_t));
    if (file_dim) *file_dim = dim;
    const uint32_t held = padded_dim(dim, multiple);
    host_matrix<Data_t, Index_t> data(num, held);   // value-initialised: the padding is zero
    if (held == dim) {
        file.read(reinterpret_cast<char*>(data.data_handle()), static_cast<std::streamsize>(data.size() * sizeof(Data_t)));
    } else {
        for (Index_t r = 0; r < num; r++) file.read(reinterpret_cast<char*>(&data(r, 0)), static_cast<std::streamsize>(dim * sizeof(Data_t)));
    }
    return data;
}

// The first `file_dim` values of every row (what load_point_data read from a file of that row length).
template <typename Data_t, typename Index_t = uint32_t>
void save_point_data(const std::string& path, host_matrix_view<const Data_t, Index_t> m, uint32_t file_dim) {
    std::ofstream file(path, std::ios::binary);
    const uint32_t num = m.extent(0);
    file.write(reinterpret_cast<const char*>(&num), sizeof(uint32_t));
    file.write(reinterpret_cast<const char*>(&file_dim), sizeof(uint32_t));
    if (file_dim == m.extent(1)) {
        file.write(reinterpret_cast<const char*>(m.data_handle()), static_cast<std::streamsize>(m.size() * sizeof(Data_t)));
    } else {
        for (Index_t r = 0; r < m.extent(0); r++) file.write(reinterpret_cast<const char*>(&m(r, 0)), static_cast<std::streamsize>(file_dim * sizeof(Data_t)));
    }
}

inline host_vector<uint32_t> load_segment_start(const std::string& path) {
    std::ifstream file(path, std::ios::binary);
    if (!file) std::cerr << "Error opening file: " << path << std::endl;
    uint32_t n = 0;
    file.read(reinterpret_cast<char*>(&n), sizeof(uint32_t));
    host_vector<uint32_t> start(n);
    file.read(reinterpret_cast<char*>(start.data_handle()), n * sizeof(uint32_t));
    return start;
}

inline host_vector<uint32_t> load_segment_length(const std::string& path) {
    std::ifstream file(path, std::ios::binary);
    if (!file) std::cerr << "Error opening file: " << path << std::endl;
    uint32_t n = 0;
    file.read(reinterpret_cast<char*>(&n), sizeof(uint32_t));
    host_vector<uint32_t> length(n);
    file.seekg(static_cast<std::streamoff>(n) * sizeof(uint32_t), std::ios::cur);
    file.read(reinterpret_cast<char*>(length.data_handle()), n * sizeof(uint32_t));
    return length;
}

inline host_vector<uint32_t> load_vector_data(const std::string& path) {
    std::ifstream file(path, std::ios::binary);
    if (!file) std::cerr << "Error opening file: " << path << std::endl;
    uint32_t n = 0;
    file.read(reinterpret_cast<char*>(&n), sizeof(uint32_t));
    host_vector<uint32_t> data(n);
    file.read(reinterpret_cast<char*>(data.data_handle()), n * sizeof(uint32_t));
    return data;
}

template <typename Data_t, typename Index_t = uint32_t>
void save_matrix_data(const std::string& path, host_matrix_view<const Data_t, Index_t> m) {
    std::ofstream file(path, std::ios::binary);
    uint32_t num = m.extent(0), dim = m.extent(1);
    file.write(reinterpret_cast<const char*>(&num), sizeof(uint32_t));
    file.write(reinterpret_cast<const char*>(&dim), sizeof(uint32_t));
    file.write(reinterpret_cast<const char*>(m.data_handle()), static_cast<std::streamsize>(m.size() * sizeof(Data_t)));
}

inline void save_segment(const std::string& path, host_vector_view<const uint32_t> start, host_vector_view<const uint32_t> length) {
    std::ofstream file(path, std::ios::binary);
    uint32_t n = start.size();
    file.write(reinterpret_cast<const char*>(&n), sizeof(uint32_t));
    file.write(reinterpret_cast<const char*>(start.data_handle()), n * sizeof(uint32_t));
    file.write(reinterpret_cast<const char*>(length.data_handle()), n * sizeof(uint32_t));
}

inline void save_vector_data(const std::string& path, host_vector_view<const uint32_t> v) {
    std::ofstream file(path, std::ios::binary);
    uint32_t n = v.size();
    file.write(reinterpret_cast<const char*>(&n), sizeof(uint32_t));
    file.write(reinterpret_cast<const char*>(v.data_handle()), n * sizeof(uint32_t));
}

}  // namespace glide
