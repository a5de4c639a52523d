// large_preprocess data_file preprocess_file result_file centroid_num sample_factor metric [boundary_factor]
// Reference: large_preprocess.cu:21-80 (same argv and output files).  With the optional boundary_factor the
// partitioning is made for a merged index (GLIDE_large::build_with_merge): the .segment file then holds one segment
// more than there are centroids, the copies of the points close to a second partition, behind all points in .reorder.  The rows may be uint8, as the reference reads them,
// or fp32; the element size is taken from the length of the data file.
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <string>

#include "load.hpp"
#include "partition_large.hpp"

using namespace glide;

template <typename Data_t>
static void run(device_resources& handle, PartitionParameter& param, const std::string& data_file, const std::string& preprocess_file,
                std::string& result_file, uint32_t batch_num) {
    uint32_t file_dim = 0;   // rows are held padded to 16 bytes (load.hpp); the files written below keep the data file's length
    auto h_data = load_points_pinned<Data_t>(data_file, &file_dim);
    const size_t num = h_data.extent(0), dim = h_data.extent(1);
    pinned_matrix<Data_t> h_reorder(num, dim);
    host_vector<uint32_t> h_map(num), h_segment_start(param.centroid_num), h_segment_length(param.centroid_num);
    device_matrix<float> d_centroids(param.centroid_num, dim);
    preprocess_for_large<Data_t>(handle, param, h_data, h_reorder, h_map.view(), h_segment_start.view(), h_segment_length.view(), d_centroids.view(),
                                batch_num, result_file);
    host_matrix<float> h_centroids(param.centroid_num, dim);
    copy_to_host(h_centroids.data_handle(), d_centroids.data_handle(), h_centroids.size());
    save_point_data<float, uint32_t>(preprocess_file + ".centroid", std::as_const(h_centroids).view(), file_dim);
    save_segment(preprocess_file + ".segment", std::as_const(h_segment_start).view(), std::as_const(h_segment_length).view());
    save_vector_data(preprocess_file + ".map", std::as_const(h_map).view());
    save_points_pinned(preprocess_file + ".reorder", h_reorder, file_dim);
}

template <typename Data_t>
static void run_merge(device_resources& handle, PartitionParameter& param, const std::string& data_file, const std::string& preprocess_file,
                      std::string& result_file, uint32_t batch_num) {
    uint32_t file_dim = 0;   // rows are held padded to 16 bytes (load.hpp); the files written below keep the data file's length
    auto h_data = load_points_pinned<Data_t>(data_file, &file_dim);
    device_matrix<float> d_centroids(param.centroid_num, h_data.extent(1));
    auto part = preprocess_for_large_merge<Data_t>(handle, param, h_data, d_centroids.view(), batch_num, result_file);
    host_matrix<float> h_centroids(param.centroid_num, h_data.extent(1));
    copy_to_host(h_centroids.data_handle(), d_centroids.data_handle(), h_centroids.size());
    save_point_data<float, uint32_t>(preprocess_file + ".centroid", std::as_const(h_centroids).view(), file_dim);
    save_segment(preprocess_file + ".segment", std::as_const(part.h_segment_start).view(), std::as_const(part.h_segment_length).view());
    save_vector_data(preprocess_file + ".map", std::as_const(part.h_map).view());
    save_points_pinned(preprocess_file + ".reorder", part.h_reorder_data, file_dim);
}

int main(int argc, char** argv) {
    if (argc != 7 && argc != 8) {
        std::cout << argv[0] << " data_file preprocess_file result_file centroid_num sample_factor metric [boundary_factor]" << std::endl;
        exit(-1);
    }
    device_resources handle(std::getenv("GLIDE_DEVICE") ? std::atoi(std::getenv("GLIDE_DEVICE")) : 0);
    std::string data_file(argv[1]), preprocess_file(argv[2]), result_file(argv[3]);
    PartitionParameter param;
    param.centroid_num = std::stoi(argv[4]);
    param.sample_factor = std::stof(argv[5]);
    std::string metric(argv[6]);
    param.metric = metric == "Cosine" ? Metric::Cosine : Metric::Euclidean;
    const uint32_t batch_num = 10;   // large_preprocess.cu:66

    std::ifstream probe(result_file);
    if (!probe.good()) {
        std::ofstream result_out(result_file, std::ios::app);
        result_out << "pre_time,knn_time,degree,index_time,beam,search_time,QPS,recall" << std::endl;
    }
    const bool bytes = fbin_element_bytes(data_file) == 1;
    if (argc == 8) {
        param.boundary_factor = std::stof(argv[7]);
        if (bytes) run_merge<uint8_t>(handle, param, data_file, preprocess_file, result_file, batch_num);
        else run_merge<float>(handle, param, data_file, preprocess_file, result_file, batch_num);
    } else {
        if (bytes) run<uint8_t>(handle, param, data_file, preprocess_file, result_file, batch_num);
        else run<float>(handle, param, data_file, preprocess_file, result_file, batch_num);
    }
    return 0;
}
