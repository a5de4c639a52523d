// File formats of the reference's load.cuh:8-128, byte for byte:
//   matrix (fbin)  u32 num, u32 dim, num*dim values            (.centroid, .reorder, knn file, .graph, data, truth)
//   segment        u32 n, u32 start[n], u32 length[n]          (.segment; n = centroid_num + 1, last = boundary)
//   vector         u32 n, u32 value[n]                         (.map, .sp)
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
