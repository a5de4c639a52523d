// large_knn preprocess_file knn_file result_file knn_degree      (reference: large_knn.cu:18-47)
#include <cstdlib>
#include <iostream>
#include <string>

#include "load.hpp"
#include "nn_descent.hpp"

using namespace glide;

// uint8 rows as in the reference (large_knn.cu:38) or fp32 rows, told apart by the length of the .reorder file
template <typename Data_t>
static void run(device_resources& handle, const std::string& preprocess_file, const std::string& knn_file, std::string& result_file,
                uint32_t knn_degree) {
    auto h_reorder = load_points_pinned<Data_t>(preprocess_file + ".reorder");
    auto h_segment_start = load_segment_start(preprocess_file + ".segment");
    auto h_segment_length = load_segment_length(preprocess_file + ".segment");
    const uint32_t iterations = std::getenv("GLIDE_NND_ITERATIONS") ? std::atoi(std::getenv("GLIDE_NND_ITERATIONS")) : 20;
    auto knn = build_knn_for_large<Data_t>(handle, knn_degree, h_segment_start.view(), h_segment_length.view(), h_reorder, result_file, iterations);
    save_matrix_pinned(knn_file, knn);
}

int main(int argc, char** argv) {
    if (argc != 5) {
        std::cout << argv[0] << " preprocess_file knn_file result_file knn_degree" << std::endl;
        exit(-1);
    }
    device_resources handle(std::getenv("GLIDE_DEVICE") ? std::atoi(std::getenv("GLIDE_DEVICE")) : 0);
    std::string preprocess_file(argv[1]), knn_file(argv[2]), result_file(argv[3]);
    const uint32_t knn_degree = std::stoi(argv[4]);
    if (fbin_element_bytes(preprocess_file + ".reorder") == 1) run<uint8_t>(handle, preprocess_file, knn_file, result_file, knn_degree);
    else run<float>(handle, preprocess_file, knn_file, result_file, knn_degree);
    return 0;
}
