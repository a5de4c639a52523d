// large_search preprocess_file query_file truth_file graph_base_file result_file metric topk beam min_graph_num boundary_factor
// Reference: large_search.cu:57-127.
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <string>

#include "glide_large.hpp"

using namespace glide;

static float calculate_recall(host_matrix<uint32_t>& result_ids, host_matrix<uint32_t>& truth, uint32_t top_k) {   // large_search.cu:14-36
    uint32_t hit = 0;
    for (uint32_t q = 0; q < result_ids.extent(0); q++)
        for (uint32_t i = 0; i < top_k; i++)
            for (uint32_t j = 0; j < top_k; j++)
                if (result_ids(q, i) == truth(q, j)) {
                    hit++;
                    break;
                }
    return static_cast<float>(hit) / (static_cast<float>(result_ids.extent(0)) * top_k);
}

int main(int argc, char** argv) {
    if (argc != 11) {
        std::cout << argv[0] << " preprocess_file query_file truth_file graph_base_file result_file metric topk beam min_graph_num boundary_factor"
                  << std::endl;
        exit(-1);
    }
    device_resources handle(std::getenv("GLIDE_DEVICE") ? std::atoi(std::getenv("GLIDE_DEVICE")) : 0);
    std::string preprocess_file(argv[1]), query_file(argv[2]), truth_file(argv[3]), graph_base_file(argv[4]), result_file(argv[5]), metric_name(argv[6]);
    std::string centroid_file = preprocess_file + ".centroid", segment_file = preprocess_file + ".segment", map_file = preprocess_file + ".map",
                reorder_file = preprocess_file + ".reorder", graph_file = graph_base_file + ".graph", sp_file = graph_base_file + ".sp";
    Metric metric = metric_name == "Cosine" ? Metric::Cosine : Metric::Euclidean;
    SearchParameter param;
    param.top_k = std::stoi(argv[7]);
    param.beam = std::stoi(argv[8]);
    const uint32_t min_segment_num = std::stoi(argv[9]);
    const float boundary_factor = std::stof(argv[10]);
    {
        std::ofstream result_out(result_file, std::ios::app);
        result_out << param.beam << ",";
    }
    auto h_truth = load_matrix_data<uint32_t, uint32_t>(truth_file);
    const uint32_t query_number = h_truth.extent(0);
    host_matrix<uint32_t> result_ids(query_number, param.top_k);
    host_matrix<float> result_dists(query_number, param.top_k);
    auto run = [&](auto tag) {   // rows and queries are uint8 as in the reference (large_search.cu:99-112) or fp32, by the .reorder file
        using Data_t = decltype(tag);
        GLIDE_large<Data_t, uint64_t> index(handle, metric, reorder_file, map_file, centroid_file, segment_file, sp_file, graph_file);
        adjust_search_params(param.min_iterations, param.max_iterations, param.beam);
        param.hash_bit = calculate_hash_bitlen(param.beam, index.graph_degree(), param.hash_max_fill_rate, param.hashmap_min_bitlen);
        param.hash_reset_interval = calculate_hash_reset_interval(param.beam, index.graph_degree(), param.hash_max_fill_rate, param.hash_bit);
        auto h_query = load_point_data<Data_t, uint32_t>(query_file);
        device_matrix<Data_t> d_query(h_query.extent(0), h_query.extent(1));
        copy_to_device(d_query.data_handle(), h_query.data_handle(), h_query.size());
        index.search(param, min_segment_num, boundary_factor, d_query.view(), result_ids.view(), result_dists.view(), result_file);
    };
    if (fbin_element_bytes(reorder_file) == 1) run(uint8_t{});
    else run(float{});
    const float recall = calculate_recall(result_ids, h_truth, param.top_k);
    std::cout << "total_recall: " << recall << std::endl;
    std::ofstream result_out(result_file, std::ios::app);
    result_out << recall << std::endl;
    return 0;
}
