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
                                param.max_iterations, param.seed, d_knn.data_handle(), ws.get(), wb, nullptr, handle.stream()),
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
