// build_nnd(): per-partition NN-descent kNN graph.  Reference: nn_descent.cuh:1405-1467 (wrapper) over
// GNND::build (:1238-1403); here the whole iteration loop runs on the device behind glide_hip_nnd_build.
#pragma once
#include <fstream>
#include <iostream>
#include <optional>
#include <string>

#include "mdarray.hpp"
#include "params.hpp"

namespace glide {

template <typename Data_t>
host_matrix<int> build_nnd(device_resources& handle, NNDescentParameter& param, std::optional<device_matrix<Data_t>>& d_data,
                           host_vector_view<uint32_t> h_segment_start_view, host_vector_view<uint32_t> h_segment_length_view,
                           std::string& result_file) {
    uint32_t graph_degree = param.graph_degree;
    if (param.intermediate_graph_degree < graph_degree) graph_degree = param.intermediate_graph_degree;   // nn_descent.cuh:1423-1425
    const uint32_t num = d_data->extent(0), dim = d_data->extent(1);
    const uint32_t segment_num = h_segment_start_view.size();
    device_vector<uint32_t> d_start(segment_num), d_length(segment_num);
    copy_to_device(d_start.data_handle(), h_segment_start_view.data_handle(), segment_num);
    copy_to_device(d_length.data_handle(), h_segment_length_view.data_handle(), segment_num);
    device_matrix<uint32_t> d_knn(num, graph_degree);
    const size_t wb = glide_hip_nnd_workspace_bytes(num, dim, graph_degree);
    device_buffer ws(wb);
    gpu_timer timer;
    timer.start();
    hip_try(glide_hip_nnd_build(d_data->data_handle(), num, dim, d_start.data_handle(), d_length.data_handle(), segment_num, graph_degree,
                                param.max_iterations, param.termination_threshold, param.seed, d_knn.data_handle(), ws.get(), wb, nullptr,
                                handle.stream()),
            "glide_hip_nnd_build");
    const float build_time = timer.stop();
    d_data.reset();   // the reference consumes the input matrix (nn_descent.cuh:1257)
    host_matrix<int> nnd_graph(num, graph_degree);
    copy_to_host(reinterpret_cast<uint32_t*>(nnd_graph.data_handle()), d_knn.data_handle(), d_knn.size());
    std::cout << "knn time: " << build_time << " s" << std::endl;
    std::ofstream result_out(result_file, std::ios::app);
    result_out << build_time << ",";
    return nnd_graph;
}

}  // namespace glide

#include "pinned.hpp"

namespace glide {

// build_knn_for_large (reference nn_descent.cuh:1515-1580 runs cuvs::neighbors::nn_descent::build per partition):
// each partition is staged from pinned host memory and its kNN graph is built by glide_hip_nnd_build as a
// single-segment problem; the next partition is copied while the current one is processed.
template <typename Data_t>
pinned_matrix<int> build_knn_for_large(device_resources& handle, uint32_t knn_degree, host_vector_view<uint32_t> h_segment_start_view,
                                       host_vector_view<uint32_t> h_segment_length_view, const pinned_matrix<Data_t>& h_reorder_data,
                                       std::string& result_file, uint32_t iterations = 20, uint32_t seed = 0,
                                       float termination_threshold = 0.0001f) {
    (void) handle;
    const uint32_t segments = h_segment_start_view.size(), dim = h_reorder_data.extent(1);
    const size_t num = h_reorder_data.extent(0);
    uint32_t max_len = 0;
    for (uint32_t s = 0; s < segments; s++) max_len = std::max(max_len, h_segment_length_view(s));
    pinned_matrix<int> knn_graph(num, knn_degree);
    staged_rows<Data_t> d_data[2] = {staged_rows<Data_t>(max_len, dim), staged_rows<Data_t>(max_len, dim)};
    device_matrix<uint32_t> d_knn[2] = {device_matrix<uint32_t>(max_len, knn_degree), device_matrix<uint32_t>(max_len, knn_degree)};
    const size_t wb = glide_hip_nnd_workspace_bytes(max_len, dim, knn_degree);
    device_buffer ws(wb);
    device_vector<uint32_t> d_seg(2 * segments);   // per partition: {start = 0, length}
    std::vector<uint32_t> h_seg(2 * segments);
    for (uint32_t s = 0; s < segments; s++) { h_seg[2 * s] = 0; h_seg[2 * s + 1] = h_segment_length_view(s); }
    copy_to_device(d_seg.data_handle(), h_seg.data(), h_seg.size());
    stager st;
    auto stage = [&](uint32_t s) {
        const int b = s & 1;
        st.before_copy(b);
        d_data[b].upload_async(h_reorder_data.row(h_segment_start_view(s)), h_segment_length_view(s), st.copy_stream());
        st.after_copy(b);
    };
    void* t0 = nullptr;
    void* t1 = nullptr;
    hip_try(glide_hip_event_create(&t0), "glide_hip_event_create");
    hip_try(glide_hip_event_create(&t1), "glide_hip_event_create");
    hip_try(glide_hip_event_record(t0, st.compute_stream()), "glide_hip_event_record");
    if (segments) stage(0);
    for (uint32_t s = 0; s < segments; s++) {
        const int b = s & 1;
        const uint32_t len = h_segment_length_view(s);
        if (s + 1 < segments) stage(s + 1);
        st.before_compute(b);
        d_data[b].widen(len, st.compute_stream());
        hip_try(glide_hip_nnd_build(d_data[b].data_handle(), len, dim, d_seg.data_handle() + 2 * s, d_seg.data_handle() + 2 * s + 1, 1, knn_degree,
                                    iterations, termination_threshold, seed + s, d_knn[b].data_handle(), ws.get(), wb, nullptr,
                                    st.compute_stream()),
                "glide_hip_nnd_build");
        hip_try(glide_hip_memcpy_d2h_async(knn_graph.row(h_segment_start_view(s)), d_knn[b].data_handle(),
                                           static_cast<size_t>(len) * knn_degree * sizeof(uint32_t), st.compute_stream()),
                "glide_hip_memcpy_d2h_async");
        st.after_compute(b);
    }
    hip_try(glide_hip_event_record(t1, st.compute_stream()), "glide_hip_event_record");
    st.sync();
    float ms = 0.f;
    hip_try(glide_hip_event_elapsed_ms(t0, t1, &ms), "glide_hip_event_elapsed_ms");
    glide_hip_event_destroy(t0);
    glide_hip_event_destroy(t1);
    const float build_time = ms / 1000.0f;   // wall time of the pipeline, copies included
    std::cout << "knn time: " << build_time << " s" << std::endl;
    std::ofstream result_out(result_file, std::ios::app);
    result_out << build_time << ",";
    return knn_graph;
}

}  // namespace glide
