// preprocess_for_large(): partitioning of a data set that lives in host memory, staged through the GPU in batches.
// Reference: partition.cuh:195-447 (get_centroids_for_large, define_partition_for_large, reorder_for_large_dataset).
// The reference's large path has no boundary list; preprocess_for_large_merge() adds one (a last segment holding a
// copy of every point that sits close to a second partition, as on the small path, partition.cuh:61-157), which is
// what GLIDE_large::build_with_merge joins the partitions with.  Rows keep their input order inside each segment.
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

// what the assignment pass leaves for the regrouping pass
struct large_partition_plan {
    uint32_t batch_num = 0, batch_size = 0;
    std::vector<std::vector<uint32_t>> batch_index;    // per batch: count x 3 {segment, slot, boundary slot}
    std::vector<std::vector<uint32_t>> batch_length;   // per batch: centroid_num + 1 counts, the last for boundary copies
    std::vector<uint32_t> total;                       // centroid_num + 1 sums over the batches
};

// get_centroids_for_large (partition.cuh:195-250): the sampled rows are gathered on the host (they are 1 % of the
// data) and clustered on the GPU.  Returns GPU seconds.
template <typename Data_t>
float get_centroids_for_large(device_resources& handle, const PartitionParameter& param, const pinned_matrix<Data_t>& h_data,
                              device_matrix_view<float> d_centroid_view) {
    const uint32_t num = h_data.extent(0), dim = h_data.extent(1), c = param.centroid_num;
    uint32_t sample_num = std::max<uint32_t>(static_cast<uint32_t>(num * param.sample_factor), std::min(num, c));
    std::vector<uint32_t> indices(num);
    std::iota(indices.begin(), indices.end(), 0u);
    std::mt19937 gen(param.seed);
    std::shuffle(indices.begin(), indices.end(), gen);
    host_matrix<float> h_sample(sample_num, dim);
    for (uint32_t i = 0; i < sample_num; i++) std::copy_n(h_data.row(indices[i]), dim, &h_sample(i, 0));   // widens uint8 rows
    device_matrix<float> d_sample(sample_num, dim);
    copy_to_device(d_sample.data_handle(), h_sample.data_handle(), h_sample.size());
    const size_t wb = glide_hip_kmeans_workspace_bytes(c, dim), sb = glide_hip_kmeans_seed_workspace_bytes(sample_num);
    device_buffer ws(wb), seed_ws(sb);
    gpu_timer timer;
    timer.start();
    hip_try(glide_hip_kmeans_seed(d_sample.data_handle(), sample_num, dim, c, param.seed, d_centroid_view.data_handle(), nullptr, seed_ws.get(), sb,
                                  handle.stream()),
            "glide_hip_kmeans_seed");
    hip_try(glide_hip_kmeans_fit(d_sample.data_handle(), sample_num, dim, c, param.kmeans_iterations, d_centroid_view.data_handle(), ws.get(), wb,
                                 handle.stream()),
            "glide_hip_kmeans_fit");
    return timer.stop();
}

// define_partition_for_large (partition.cuh:252-337): per batch, nearest centroid + slot inside the batch; the
// lengths accumulate on the host.  boundary_factor 0 marks no boundary copies (the reference's large path).
template <typename Data_t>
float define_partition_for_large(device_resources& handle, const PartitionParameter& param, float boundary_factor,
                                 const pinned_matrix<Data_t>& h_data, device_matrix_view<float> d_centroid_view, uint32_t batch_num,
                                 large_partition_plan& plan) {
    const uint32_t num = h_data.extent(0), dim = h_data.extent(1), c = param.centroid_num;
    if (batch_num == 0) batch_num = 1;
    const uint32_t batch_size = (num + batch_num - 1) / batch_num;
    plan.batch_num = batch_num;
    plan.batch_size = batch_size;
    plan.batch_index.assign(batch_num, {});
    plan.batch_length.assign(batch_num, std::vector<uint32_t>(c + 1, 0));
    plan.total.assign(c + 1, 0);
    staged_rows<Data_t> d_batch(batch_size, dim);
    device_matrix<uint32_t> d_segment_index(batch_size, 3);
    device_vector<uint32_t> d_batch_length(c + 1);
    const size_t wb = glide_hip_partition_assign_workspace_bytes(batch_size, c);
    device_buffer ws(wb);
    gpu_timer timer;
    float seconds = 0.0f;
    for (uint32_t b = 0; b < batch_num; b++) {
        const uint32_t first = b * batch_size;
        if (first >= num) break;
        const uint32_t count = std::min(batch_size, num - first);
        copy_to_device(d_batch.stored(), h_data.row(first), static_cast<size_t>(count) * dim);
        d_batch.widen(count, handle.stream());
        timer.start();
        hip_try(glide_hip_partition_assign(d_batch.data_handle(), count, dim, d_centroid_view.data_handle(), c, boundary_factor,
                                           metric_code(param.metric), d_segment_index.data_handle(), d_batch_length.data_handle(), nullptr, ws.get(),
                                           wb, handle.stream()),
                "glide_hip_partition_assign");
        seconds += timer.stop();
        plan.batch_index[b].resize(static_cast<size_t>(count) * 3);
        copy_to_host(plan.batch_index[b].data(), d_segment_index.data_handle(), plan.batch_index[b].size());
        copy_to_host(plan.batch_length[b].data(), d_batch_length.data_handle(), c + 1);
        for (uint32_t s = 0; s <= c; s++) plan.total[s] += plan.batch_length[b][s];
    }
    return seconds;
}

// reorder_for_large_dataset (partition.cuh:339-415): each batch is grouped by segment on the GPU, then each group is
// copied to its place.  Rows move in their stored type: the regrouping kernel only copies bits, so a uint8 row of
// `dim` bytes is handed to it as dim / 4 32-bit words.  h_segment_start has centroid_num entries, or centroid_num + 1
// when the plan holds boundary copies; their group follows the batch's own rows in the staging buffer and lands
// behind the last partition (rows num..).
template <typename Data_t>
float reorder_for_large_dataset(device_resources& handle, const pinned_matrix<Data_t>& h_data, const large_partition_plan& plan,
                                uint32_t centroid_num, pinned_matrix<Data_t>& h_reorder_data, host_vector_view<uint32_t> h_map_view,
                                host_vector_view<uint32_t> h_segment_start_view) {
    const uint32_t num = h_data.extent(0), dim = h_data.extent(1), c = centroid_num;
    const bool with_boundary = h_segment_start_view.size() == c + 1;
    const uint32_t groups = with_boundary ? c + 1 : c;
    if (sizeof(Data_t) == 1 && dim % 16 != 0) throw std::invalid_argument("uint8 rows need dim % 16 == 0");
    const uint32_t words = dim * sizeof(Data_t) / 4;
    uint32_t max_out = plan.batch_size;
    if (with_boundary)
        for (uint32_t b = 0; b < plan.batch_num; b++) max_out = std::max(max_out, plan.batch_size + plan.batch_length[b][c]);
    staged_rows<Data_t> d_batch(plan.batch_size, dim);
    device_matrix<uint32_t> d_segment_index(plan.batch_size, 3);
    device_buffer d_grouped(static_cast<size_t>(max_out) * dim * sizeof(Data_t) + 16);
    device_vector<uint32_t> d_batch_map(max_out), d_batch_start(c + 1);
    std::vector<uint32_t> filled(c + 1, 0), batch_start(c + 1);
    std::vector<uint32_t> h_batch_map(max_out);
    gpu_timer timer;
    float seconds = 0.0f;
    for (uint32_t b = 0; b < plan.batch_num; b++) {
        const uint32_t first = b * plan.batch_size;
        if (first >= num) break;
        const uint32_t count = std::min(plan.batch_size, num - first);
        uint32_t run = 0;
        for (uint32_t s = 0; s <= c; s++) {
            batch_start[s] = run;   // batch_start[c] == count: where the batch's boundary copies begin
            if (s < c) run += plan.batch_length[b][s];
        }
        copy_to_device(d_batch.stored(), h_data.row(first), static_cast<size_t>(count) * dim);
        copy_to_device(d_segment_index.data_handle(), plan.batch_index[b].data(), plan.batch_index[b].size());
        copy_to_device(d_batch_start.data_handle(), batch_start.data(), c + 1);
        timer.start();
        hip_try(glide_hip_reorder_batch(reinterpret_cast<const float*>(d_batch.stored()), count, words, d_segment_index.data_handle(),
                                        d_batch_start.data_handle(), first, static_cast<float*>(d_grouped.get()), d_batch_map.data_handle(),
                                        handle.stream()),
                "glide_hip_reorder_batch");
        seconds += timer.stop();
        const uint32_t out_rows = count + (with_boundary ? plan.batch_length[b][c] : 0);
        copy_to_host(h_batch_map.data(), d_batch_map.data_handle(), out_rows);
        for (uint32_t s = 0; s < groups; s++) {
            const uint32_t len = plan.batch_length[b][s];
            if (!len) continue;
            const size_t dst_row = static_cast<size_t>(h_segment_start_view(s)) + filled[s];
            copy_to_host(h_reorder_data.row(dst_row), static_cast<const Data_t*>(d_grouped.get()) + static_cast<size_t>(batch_start[s]) * dim,
                         static_cast<size_t>(len) * dim);
            std::copy_n(h_batch_map.data() + batch_start[s], len, h_map_view.data_handle() + dst_row);
            filled[s] += len;
        }
    }
    return seconds;
}

inline void report_preprocess_time(float build_time, std::string& result_file) {
    std::cout << "preprocessing time: " << build_time << " s" << std::endl;
    std::ofstream result_out(result_file, std::ios::app);
    result_out << build_time << ",";
}

// partition.cuh:417-447
template <typename Data_t>
void preprocess_for_large(device_resources& handle, PartitionParameter param, const pinned_matrix<Data_t>& h_data,
                          pinned_matrix<Data_t>& h_reorder_data, host_vector_view<uint32_t> h_map_view,
                          host_vector_view<uint32_t> h_segment_start_view, host_vector_view<uint32_t> h_segment_length_view,
                          device_matrix_view<float> d_centroid_view, uint32_t batch_num, std::string& result_file) {
    const uint32_t c = param.centroid_num;
    float build_time = get_centroids_for_large(handle, param, h_data, d_centroid_view);
    large_partition_plan plan;
    build_time += define_partition_for_large(handle, param, 0.0f, h_data, d_centroid_view, batch_num, plan);
    uint32_t start = 0;
    for (uint32_t s = 0; s < c; s++) {
        h_segment_start_view(s) = start;
        h_segment_length_view(s) = plan.total[s];
        start += plan.total[s];
    }
    build_time += reorder_for_large_dataset(handle, h_data, plan, c, h_reorder_data, h_map_view, h_segment_start_view);
    report_preprocess_time(build_time, result_file);
}

// Partitioning for a merged large index: centroid_num + 1 segments, the last one holding the boundary copies
// (param.boundary_factor, as define_partition on the small path).  The outputs are sized here because the number of
// copies is only known after the assignment pass.
template <typename Data_t>
struct large_merge_partition {
    pinned_matrix<Data_t> h_reorder_data;                    // (num + copies) x dim
    host_vector<uint32_t> h_map, h_segment_start, h_segment_length;
};

template <typename Data_t>
large_merge_partition<Data_t> preprocess_for_large_merge(device_resources& handle, PartitionParameter param, const pinned_matrix<Data_t>& h_data,
                                                         device_matrix_view<float> d_centroid_view, uint32_t batch_num, std::string& result_file) {
    const uint32_t num = h_data.extent(0), dim = h_data.extent(1), c = param.centroid_num;
    float build_time = get_centroids_for_large(handle, param, h_data, d_centroid_view);
    large_partition_plan plan;
    build_time += define_partition_for_large(handle, param, param.boundary_factor, h_data, d_centroid_view, batch_num, plan);
    const size_t rows = static_cast<size_t>(num) + plan.total[c];
    if (rows >= 0x7fffffffull) throw std::invalid_argument("more than 2^31 - 1 reorder rows");
    large_merge_partition<Data_t> out{pinned_matrix<Data_t>(rows, dim), host_vector<uint32_t>(rows), host_vector<uint32_t>(c + 1),
                                      host_vector<uint32_t>(c + 1)};
    uint32_t start = 0;
    for (uint32_t s = 0; s <= c; s++) {
        out.h_segment_start(s) = start;
        out.h_segment_length(s) = plan.total[s];
        start += plan.total[s];
    }
    build_time += reorder_for_large_dataset(handle, h_data, plan, c, out.h_reorder_data, out.h_map.view(), out.h_segment_start.view());
    report_preprocess_time(build_time, result_file);
    return out;
}

}  // namespace glide
