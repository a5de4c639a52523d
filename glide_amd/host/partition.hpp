// preprocess(): centroids on a sample, partition assignment, reorder.  Reference: partition.cuh:8-193.
#pragma once
#include <algorithm>
#include <fstream>
#include <iostream>
#include <numeric>
#include <optional>
#include <random>
#include <string>
#include <vector>

#include "mdarray.hpp"
#include "params.hpp"

namespace glide {

// get_centroids (partition.cuh:8-59): shuffle ids, gather a sample, cluster it.  The reference calls
// cuvs::cluster::kmeans::fit; here greedy k-means++ seeding, then Lloyd iterations.
template <typename Data_t, typename Index_t>
void get_centroids(device_resources& handle, device_matrix_view<Data_t, Index_t> d_data_view, device_matrix_view<float> d_centroid_view,
                   const PartitionParameter& param, float& build_time) {
    const uint32_t num = d_data_view.extent(0), dim = d_data_view.extent(1), c = param.centroid_num;
    uint32_t sample_num = std::max<uint32_t>(static_cast<uint32_t>(num * param.sample_factor), std::min(num, c));
    std::vector<uint32_t> indices(num);
    std::iota(indices.begin(), indices.end(), 0u);
    std::mt19937 gen(param.seed);
    std::shuffle(indices.begin(), indices.end(), gen);
    device_vector<uint32_t> d_indices(sample_num);
    copy_to_device(d_indices.data_handle(), indices.data(), sample_num);
    device_matrix<float> d_sample(sample_num, dim);
    const size_t wb = glide_hip_kmeans_workspace_bytes(c, dim), sb = glide_hip_kmeans_seed_workspace_bytes(sample_num);
    device_buffer ws(wb), seed_ws(sb);
    gpu_timer timer;
    timer.start();
    hip_try(glide_hip_sample_rows(d_data_view.data_handle(), dim, d_indices.data_handle(), sample_num, d_sample.data_handle(), handle.stream()),
            "glide_hip_sample_rows");
    hip_try(glide_hip_kmeans_seed(d_sample.data_handle(), sample_num, dim, c, param.seed, d_centroid_view.data_handle(), nullptr, seed_ws.get(), sb,
                                  handle.stream()),
            "glide_hip_kmeans_seed");
    hip_try(glide_hip_kmeans_fit(d_sample.data_handle(), sample_num, dim, c, param.kmeans_iterations, d_centroid_view.data_handle(), ws.get(), wb,
                                 handle.stream()),
            "glide_hip_kmeans_fit");
    build_time += timer.stop();
}

// define_partition (partition.cuh:61-116)
template <typename Data_t, typename Index_t>
void define_partition(device_resources& handle, device_matrix_view<Data_t, Index_t> d_data_view, device_matrix_view<float> d_centroid_view,
                      host_vector_view<uint32_t> h_segment_start_view, host_vector_view<uint32_t> h_segment_length_view,
                      device_matrix_view<uint32_t> d_segment_index_view, float boundary_fact, Metric metric, float& build_time) {
    const uint32_t centroid_num = d_centroid_view.extent(0), num = d_data_view.extent(0), dim = d_data_view.extent(1);
    device_vector<uint32_t> d_segment_length(h_segment_length_view.size());
    const size_t wb = glide_hip_partition_assign_workspace_bytes(num, centroid_num);
    device_buffer ws(wb);
    gpu_timer timer;
    timer.start();
    hip_try(glide_hip_partition_assign(d_data_view.data_handle(), num, dim, d_centroid_view.data_handle(), centroid_num, boundary_fact,
                                       metric_code(metric), d_segment_index_view.data_handle(), d_segment_length.data_handle(), nullptr,
                                       ws.get(), wb, handle.stream()),
            "glide_hip_partition_assign");
    build_time += timer.stop();
    copy_to_host(h_segment_length_view.data_handle(), d_segment_length.data_handle(), d_segment_length.size());
    uint32_t start = 0;
    for (uint32_t i = 0; i < h_segment_length_view.size(); i++) {
        h_segment_start_view(i) = start;
        start += h_segment_length_view(i);
    }
}

// reorder (partition.cuh:118-157)
template <typename Data_t, typename Index_t>
void reorder(device_resources& handle, device_matrix_view<Data_t, Index_t> d_data_view, device_vector_view<uint32_t> d_map_view,
             device_matrix_view<Data_t, Index_t> d_reorder_data_view, host_vector_view<uint32_t> h_segment_start_view,
             device_matrix_view<uint32_t> d_segment_index_view, float& build_time) {
    const uint32_t num = d_data_view.extent(0), dim = d_data_view.extent(1);
    device_vector<uint32_t> d_segment_start(h_segment_start_view.size());
    copy_to_device(d_segment_start.data_handle(), h_segment_start_view.data_handle(), h_segment_start_view.size());
    gpu_timer timer;
    timer.start();
    hip_try(glide_hip_reorder(d_data_view.data_handle(), num, dim, d_segment_index_view.data_handle(), d_segment_start.data_handle(),
                              d_reorder_data_view.data_handle(), d_map_view.data_handle(), handle.stream()),
            "glide_hip_reorder");
    build_time += timer.stop();
}

// preprocess (partition.cuh:159-193); h_segment_*_view have centroid_num + 1 entries
template <typename Data_t, typename Index_t>
void preprocess(device_resources& handle, PartitionParameter param, device_matrix_view<Data_t, Index_t> d_data_view,
                std::optional<device_matrix<Data_t, Index_t>>& d_reorder_data, std::optional<device_vector<uint32_t>>& d_map,
                host_vector_view<uint32_t> h_segment_start_view, host_vector_view<uint32_t> h_segment_length_view,
                device_matrix_view<float> d_centroid_view, std::string& result_file) {
    const uint32_t num = d_data_view.extent(0), dim = d_data_view.extent(1);
    float build_time = 0.0f;
    device_matrix<uint32_t> d_segment_index(num, 3);
    get_centroids<Data_t, Index_t>(handle, d_data_view, d_centroid_view, param, build_time);
    define_partition<Data_t, Index_t>(handle, d_data_view, d_centroid_view, h_segment_start_view, h_segment_length_view,
                                      d_segment_index.view(), param.boundary_factor, param.metric, build_time);
    const uint32_t reorder_num = num + h_segment_length_view(param.centroid_num);
    d_reorder_data.emplace(reorder_num, dim);
    d_map.emplace(reorder_num);
    reorder<Data_t, Index_t>(handle, d_data_view, d_map->view(), d_reorder_data->view(), h_segment_start_view, d_segment_index.view(),
                             build_time);
    std::cout << "preprocessing time: " << build_time << " s" << std::endl;
    std::ofstream result_out(result_file, std::ios::app);
    result_out << build_time << ",";
}

}  // namespace glide
