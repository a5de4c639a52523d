// small_build data_file preprocess_file knn_file graph_base_file result_file metric graph_degree knn_degree relaxant_factor beam refine_beam
// Reference: small_build.cu:25-136 (same argv; writes <graph_base>.graph and <graph_base>.sp).
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <optional>
#include <string>

#include "glide.hpp"
#include "load.hpp"

using namespace glide;

int main(int argc, char** argv) {
    if (argc != 12) {
        std::cout << argv[0]
                  << "data_file preprocess_file knn_file graph_base_file result_file metric graph_degree knn_degree relaxant_factor beam refine_beam"
                  << std::endl;
        exit(-1);
    }
    device_resources handle(std::getenv("GLIDE_DEVICE") ? std::atoi(std::getenv("GLIDE_DEVICE")) : 0);
    std::string data_file(argv[1]), preprocess_file(argv[2]), knn_file(argv[3]), graph_base_file(argv[4]), result_file(argv[5]), metric(argv[6]);

    IndexParameter build_param;
    build_param.graph_degree = std::stoi(argv[7]);
    build_param.knn_degree = std::stoi(argv[8]);
    build_param.relaxant_factor = std::stof(argv[9]);
    if (metric == "Euclidean") build_param.metric = Metric::Euclidean;
    else if (metric == "Cosine") build_param.metric = Metric::Cosine;

    auto size_param = [&](SearchParameter& p, uint32_t beam) {   // small_build.cu:61-82 (both sized with knn_degree)
        p.beam = beam;
        adjust_search_params(p.min_iterations, p.max_iterations, p.beam);
        p.hash_bit = calculate_hash_bitlen(p.beam, build_param.knn_degree, p.hash_max_fill_rate, p.hashmap_min_bitlen);
        p.hash_reset_interval = calculate_hash_reset_interval(p.beam, build_param.knn_degree, p.hash_max_fill_rate, p.hash_bit);
    };
    SearchParameter search_param_knn, search_param_refine;
    size_param(search_param_knn, std::stoi(argv[10]));
    search_param_refine.beam = std::stoi(argv[11]);
    if (search_param_refine.beam != 0) size_param(search_param_refine, search_param_refine.beam);

    auto h_data = load_point_data<float, uint32_t>(data_file);
    auto h_centroids = load_point_data<float, uint32_t>(preprocess_file + ".centroid");
    auto h_segment_start = load_segment_start(preprocess_file + ".segment");
    auto h_segment_length = load_segment_length(preprocess_file + ".segment");
    auto h_map = load_vector_data(preprocess_file + ".map");
    auto h_reorder_data = load_point_data<float, uint32_t>(preprocess_file + ".reorder");
    auto h_knn_graph = load_matrix_data<uint32_t, uint32_t>(knn_file);

    std::optional<device_matrix<float, uint32_t>> d_reorder_data;
    std::optional<device_vector<uint32_t>> d_map, d_segment_start, d_segment_length;
    std::optional<device_matrix<uint32_t, uint32_t>> d_knn_graph;
    d_reorder_data.emplace(h_reorder_data.extent(0), h_reorder_data.extent(1));
    d_map.emplace(h_map.size());
    d_segment_start.emplace(h_segment_start.size());
    d_segment_length.emplace(h_segment_length.size());
    d_knn_graph.emplace(h_knn_graph.extent(0), h_knn_graph.extent(1));
    copy_to_device(d_reorder_data->data_handle(), h_reorder_data.data_handle(), h_reorder_data.size());
    copy_to_device(d_map->data_handle(), h_map.data_handle(), h_map.size());
    copy_to_device(d_segment_start->data_handle(), h_segment_start.data_handle(), h_segment_start.size());
    copy_to_device(d_segment_length->data_handle(), h_segment_length.data_handle(), h_segment_length.size());
    copy_to_device(d_knn_graph->data_handle(), h_knn_graph.data_handle(), h_knn_graph.size());

    GLIDE<float, uint32_t> index(handle, build_param.graph_degree, h_data.view(), h_centroids.view(), build_param.metric);
    {
        std::ofstream result_out(result_file, std::ios::app);
        result_out << build_param.graph_degree << ",";
    }
    index.build(build_param, search_param_knn, search_param_refine, d_knn_graph, d_segment_start, d_segment_length, d_map,
                h_segment_start.view(), h_segment_length.view(), h_map.view(), d_reorder_data, result_file);

    host_matrix<uint32_t> graph(index.num(), index.graph_degree());
    copy_to_host(graph.data_handle(), index.graph_view().data_handle(), graph.size());
    host_vector<uint32_t> start_point(index.start_point_num());
    copy_to_host(start_point.data_handle(), index.start_point_view().data_handle(), start_point.size());
    save_matrix_data<uint32_t, uint32_t>(graph_base_file + ".graph", std::as_const(graph).view());
    save_vector_data(graph_base_file + ".sp", std::as_const(start_point).view());
    return 0;
}
