// small_search data_file query_file truth_file preprocess_file graph_base_file result_file metric topk beam
// Reference: small_search.cu:14-126 (calculate_recall :14-36; sizing :102-108).
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <string>

#include "glide.hpp"
#include "load.hpp"

using namespace glide;

// small_search.cu:14-36: hits among the first top_k truth entries / (query_num * top_k)
static float calculate_recall(host_matrix<uint32_t>& result_ids, host_matrix<uint32_t>& truth, uint32_t top_k) {
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
    if (argc != 10) {
        std::cout << argv[0] << " data_file query_file truth_file preprocess_file graph_base_file result_file metric topk beam" << std::endl;
        exit(-1);
    }
    device_resources handle(std::getenv("GLIDE_DEVICE") ? std::atoi(std::getenv("GLIDE_DEVICE")) : 0);
    std::string data_file(argv[1]), query_file(argv[2]), truth_file(argv[3]), preprocess_file(argv[4]), graph_base_file(argv[5]),
        result_file(argv[6]), metric_name(argv[7]);
    Metric metric = metric_name == "Cosine" ? Metric::Cosine : Metric::Euclidean;

    auto h_data = load_point_data<float, uint32_t>(data_file);
    auto h_query = load_point_data<float, uint32_t>(query_file);
    auto h_truth = load_matrix_data<uint32_t, uint32_t>(truth_file);
    auto h_centroids = load_point_data<float, uint32_t>(preprocess_file + ".centroid");
    auto h_graph = load_matrix_data<uint32_t, uint32_t>(graph_base_file + ".graph");
    auto h_start_points = load_vector_data(graph_base_file + ".sp");

    SearchParameter param;
    param.top_k = std::stoi(argv[8]);
    param.beam = std::stoi(argv[9]);
    {
        std::ofstream result_out(result_file, std::ios::app);
        result_out << param.beam << ",";
    }
    adjust_search_params(param.min_iterations, param.max_iterations, param.beam);
    param.hash_bit = calculate_hash_bitlen(param.beam, h_graph.extent(1), param.hash_max_fill_rate, param.hashmap_min_bitlen);
    param.hash_reset_interval = calculate_hash_reset_interval(param.beam, h_graph.extent(1), param.hash_max_fill_rate, param.hash_bit);

    GLIDE<float, uint32_t> index(handle, h_graph.extent(1), h_data.view(), h_centroids.view(), metric);
    index.load(h_graph.view(), h_start_points.view());

    device_matrix<float> d_query(h_query.extent(0), h_query.extent(1));
    copy_to_device(d_query.data_handle(), h_query.data_handle(), h_query.size());
    host_matrix<uint32_t> result_ids(h_query.extent(0), param.top_k);
    host_matrix<float> result_dists(h_query.extent(0), param.top_k);
    index.search(param, d_query.view(), result_ids, result_dists, result_file);

    const float recall = calculate_recall(result_ids, h_truth, param.top_k);
    std::cout << "total_recall: " << recall << std::endl;
    std::ofstream result_out(result_file, std::ios::app);
    result_out << recall << std::endl;
    return 0;
}
