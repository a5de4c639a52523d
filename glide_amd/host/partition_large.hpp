// preprocess_for_large(): partitioning of a data set that lives in host memory, staged through the GPU in batches.
// Reference: partition.cuh:195-447 (get_centroids_for_large, define_partition_for_large, reorder_for_large_dataset).
// No boundary list on this path.  Rows keep their input order inside each partition.
#pragma once
#include <algorithm>
#include <fstream>
#include <iostream>
#include <numeric>
#include <random>
#include <stdexcept>
#include <string>
#include <vector>

#include "mdarray.hpp"
#include "params.hpp"
#include "pinned.hpp"

namespace glide {

template <typename Data_t>
void preprocess_for_large(device_resources& handle, PartitionParameter param, const pinned_matrix<Data_t>& h_data,
                          pinned_matrix<Data_t>& h_reorder_data, host_vector_view<uint32_t> h_map_view,
                          host_vector_view<uint32_t> h_segment_start_view, host_vector_view<uint32_t> h_segment_length_view,
                          device_matrix_view<float> d_centroid_view, uint32_t batch_num, std::string& result_file) {
    const uint32_t num = h_data.extent(0), dim = h_data.extent(1), c = param.centroid_num;
    if (batch_num == 0) batch_num = 1;
    const uint32_t batch_size = (num + batch_num - 1) / batch_num;
    float build_time = 0.0f;
    gpu_timer timer;

    // get_centroids_for_large: the sampled rows are gathered on the host (they are 1 % of the data), clustered on the GPU
    uint32_t sample_num = std::max<uint32_t>(static_cast<uint32_t>(num * param.sample_factor), std::min(num, c));
    std::vector<uint32_t> indices(num);
    std::iota(indices.begin(), indices.end(), 0u);
    std::mt19937 gen(param.seed);
    std::shuffle(indices.begin(), indices.end(), gen);
    {
        host_matrix<float> h_sample(sample_num, dim);
        for (uint32_t i = 0; i < sample_num; i++) std::copy_n(h_data.row(indices[i]), dim, &h_sample(i, 0));   // widens uint8 rows
        device_matrix<float> d_sample(sample_num, dim);
        copy_to_device(d_sample.data_handle(), h_sample.data_handle(), h_sample.size());
        copy_to_device(d_centroid_view.data_handle(), h_sample.data_handle(), static_cast<size_t>(std::min(c, sample_num)) * dim);
        const size_t wb = glide_hip_kmeans_workspace_bytes(c, dim);
        device_buffer ws(wb);
        timer.start();
        hip_try(glide_hip_kmeans_fit(d_sample.data_handle(), sample_num, dim, c, param.kmeans_iterations, d_centroid_view.data_handle(), ws.get(),
                                     wb, handle.stream()),
                "glide_hip_kmeans_fit");
        build_time += timer.stop();
    }

    // define_partition_for_large: per batch, nearest centroid + slot inside the batch; lengths accumulate on the host
    staged_rows<Data_t> d_batch(batch_size, dim);
    device_matrix<uint32_t> d_segment_index(batch_size, 3);
    device_vector<uint32_t> d_batch_length(c + 1);
    const size_t wb = glide_hip_partition_assign_workspace_bytes(batch_size, c);
    device_buffer ws(wb);
    std::vector<std::vector<uint32_t>> batch_index(batch_num);
    std::vector<std::vector<uint32_t>> batch_length(batch_num, std::vector<uint32_t>(c + 1, 0));
    std::vector<uint32_t> total(c + 1, 0);
    for (uint32_t b = 0; b < batch_num; b++) {
        const uint32_t first = b * batch_size;
        if (first >= num) break;
        const uint32_t count = std::min(batch_size, num - first);
        copy_to_device(d_batch.stored(), h_data.row(first), static_cast<size_t>(count) * dim);
        d_batch.widen(count, handle.stream());
        timer.start();
        hip_try(glide_hip_partition_assign(d_batch.data_handle(), count, dim, d_centroid_view.data_handle(), c, 0.0f, metric_code(param.metric),
                                           d_segment_index.data_handle(), d_batch_length.data_handle(), nullptr, ws.get(), wb, handle.stream()),
                "glide_hip_partition_assign");
        build_time += timer.stop();
        batch_index[b].resize(static_cast<size_t>(count) * 3);
        copy_to_host(batch_index[b].data(), d_segment_index.data_handle(), batch_index[b].size());
        copy_to_host(batch_length[b].data(), d_batch_length.data_handle(), c + 1);
        for (uint32_t s = 0; s < c; s++) total[s] += batch_length[b][s];
    }
    uint32_t start = 0;
    for (uint32_t s = 0; s < c; s++) {
        h_segment_start_view(s) = start;
        h_segment_length_view(s) = total[s];
        start += total[s];
    }

    // reorder_for_large_dataset: each batch is grouped by segment on the GPU, then each group is copied to its place.
    // Rows move in their stored type: the regrouping kernel only copies bits, so a uint8 row of `dim` bytes is handed
    // to it as dim / 4 32-bit words.
    if (sizeof(Data_t) == 1 && dim % 16 != 0) throw std::invalid_argument("uint8 rows need dim % 16 == 0");
    const uint32_t words = dim * sizeof(Data_t) / 4;
    device_buffer d_grouped(static_cast<size_t>(batch_size) * dim * sizeof(Data_t) + 16);
    device_vector<uint32_t> d_batch_map(batch_size), d_batch_start(c + 1);
    std::vector<uint32_t> filled(c, 0), batch_start(c + 1);
    std::vector<uint32_t> h_batch_map(batch_size);
    for (uint32_t b = 0; b < batch_num; b++) {
        const uint32_t first = b * batch_size;
        if (first >= num) break;
        const uint32_t count = std::min(batch_size, num - first);
        uint32_t run = 0;
        for (uint32_t s = 0; s <= c; s++) {
            batch_start[s] = run;
            if (s < c) run += batch_length[b][s];
        }
        copy_to_device(d_batch.stored(), h_data.row(first), static_cast<size_t>(count) * dim);
        copy_to_device(d_segment_index.data_handle(), batch_index[b].data(), batch_index[b].size());
        copy_to_device(d_batch_start.data_handle(), batch_start.data(), c + 1);
        timer.start();
        hip_try(glide_hip_reorder_batch(reinterpret_cast<const float*>(d_batch.stored()), count, words, d_segment_index.data_handle(),
                                        d_batch_start.data_handle(), first, static_cast<float*>(d_grouped.get()), d_batch_map.data_handle(),
                                        handle.stream()),
                "glide_hip_reorder_batch");
        build_time += timer.stop();
        copy_to_host(h_batch_map.data(), d_batch_map.data_handle(), count);
        for (uint32_t s = 0; s < c; s++) {
            const uint32_t len = batch_length[b][s];
            if (!len) continue;
            const size_t dst_row = static_cast<size_t>(h_segment_start_view(s)) + filled[s];
            copy_to_host(h_reorder_data.row(dst_row), static_cast<const Data_t*>(d_grouped.get()) + static_cast<size_t>(batch_start[s]) * dim,
                         static_cast<size_t>(len) * dim);
            std::copy_n(h_batch_map.data() + batch_start[s], len, h_map_view.data_handle() + dst_row);
            filled[s] += len;
        }
    }
    std::cout << "preprocessing time: " << build_time << " s" << std::endl;
    std::ofstream result_out(result_file, std::ios::app);
    result_out << build_time << ",";
}

}  // namespace glide
