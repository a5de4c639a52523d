// large_build preprocess_file knn_file graph_base_file result_file metric graph_degree knn_degree relaxant_factor beam refine_beam
// Reference: large_build.cu:24-95.  A partitioning that carries a boundary segment (large_preprocess with a
// boundary_factor) is built with GLIDE_large::build_with_merge.
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <string>

#include "glide_large.hpp"

using namespace glide;

int main(int argc, char** argv) {
    if (argc != 11) {
        std::cout << argv[0] << " preprocess_file knn_file graph_base_file result_file metric graph_degree knn_degree relaxant_factor beam refine_beam"
                  << std::endl;
        exit(-1);
    }
    device_resources handle(std::getenv("GLIDE_DEVICE") ? std::atoi(std::getenv("GLIDE_DEVICE")) : 0);
    std::string preprocess_file(argv[1]), knn_file(argv[2]), graph_base_file(argv[3]), result_file(argv[4]), metric(argv[5]);
    std::string centroid_file = preprocess_file + ".centroid", segment_file = preprocess_file + ".segment", map_file = preprocess_file + ".map",
                reorder_file = preprocess_file + ".reorder";
    IndexParameter build_param;
    build_param.graph_degree = std::stoi(argv[6]);
    build_param.knn_degree = std::stoi(argv[7]);
    build_param.relaxant_factor = std::stof(argv[8]);
    build_param.metric = metric == "Cosine" ? Metric::Cosine : Metric::Euclidean;
    auto size_param = [&](SearchParameter& p, uint32_t beam) {   // large_build.cu:58-80
        p.beam = beam;
        adjust_search_params(p.min_iterations, p.max_iterations, p.beam);
        p.hash_bit = calculate_hash_bitlen(p.beam, build_param.knn_degree, p.hash_max_fill_rate, p.hashmap_min_bitlen);
        p.hash_reset_interval = calculate_hash_reset_interval(p.beam, build_param.knn_degree, p.hash_max_fill_rate, p.hash_bit);
    };
    SearchParameter search_param_knn, search_param_refine;
    size_param(search_param_knn, std::stoi(argv[9]));
    search_param_refine.beam = std::stoi(argv[10]);
    if (search_param_refine.beam != 0) size_param(search_param_refine, search_param_refine.beam);

    auto h_knn_graph = load_matrix_pinned<uint32_t>(knn_file);
    {
        std::ofstream result_out(result_file, std::ios::app);
        result_out << build_param.graph_degree << ",";
    }
    auto run = [&](auto tag) {   // uint8 rows as in the reference (large_build.cu:84) or fp32 rows, by the length of the .reorder file
        using Data_t = decltype(tag);
        GLIDE_large<Data_t, uint64_t> index(handle, build_param.graph_degree, build_param.metric, reorder_file, map_file, centroid_file, segment_file);
        if (index.merged()) index.build_with_merge(build_param, search_param_knn, search_param_refine, h_knn_graph, result_file);
        else index.build(build_param, search_param_knn, search_param_refine, h_knn_graph, result_file);
        save_matrix_pinned(graph_base_file + ".graph", index.graph_view());
        save_vector_data(graph_base_file + ".sp", index.start_point_view());
    };
    if (fbin_element_bytes(reorder_file) == 1) run(uint8_t{});
    else run(float{});
    return 0;
}
