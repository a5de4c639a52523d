// small_knn preprocess_file knn_file result_file knn_degree
// Reference: small_knn.cu:18-52.  GLIDE_NND_ITERATIONS overrides the iteration count (default 20, params.cuh:20).
#include <cstdlib>
#include <iostream>
#include <optional>
#include <string>

#include "load.hpp"
#include "nn_descent.hpp"

using namespace glide;

int main(int argc, char** argv) {
    if (argc != 5) {
        std::cout << argv[0] << " preprocess_file knn_file result_file knn_degree" << std::endl;
        exit(-1);
    }
    device_resources handle(std::getenv("GLIDE_DEVICE") ? std::atoi(std::getenv("GLIDE_DEVICE")) : 0);
    std::string preprocess_file(argv[1]), knn_file(argv[2]), result_file(argv[3]);
    const uint32_t knn_degree = std::stoi(argv[4]);

    auto h_reorder = load_point_data<float, uint32_t>(preprocess_file + ".reorder");
    auto h_segment_start = load_segment_start(preprocess_file + ".segment");
    auto h_segment_length = load_segment_length(preprocess_file + ".segment");
    std::optional<device_matrix<float>> d_data;
    d_data.emplace(h_reorder.extent(0), h_reorder.extent(1));
    copy_to_device(d_data->data_handle(), h_reorder.data_handle(), h_reorder.size());

    NNDescentParameter param(knn_degree);
    if (const char* it = std::getenv("GLIDE_NND_ITERATIONS")) param.max_iterations = std::atoi(it);
    auto knn = build_nnd<float>(handle, param, d_data, h_segment_start.view(), h_segment_length.view(), result_file);
    save_matrix_data<int, uint32_t>(knn_file, std::as_const(knn).view());
    return 0;
}
