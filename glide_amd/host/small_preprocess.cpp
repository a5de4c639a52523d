// small_preprocess data_file preprocess_file result_file centroid_num boundary_factor sample_factor metric
// Reference: small_preprocess.cu:22-89 (same argv, same output files: .centroid .segment .map .reorder).
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <optional>
#include <string>

#include "load.hpp"
#include "partition.hpp"

using namespace glide;

int main(int argc, char** argv) {
    if (argc != 8) {
        std::cout << argv[0] << " data_file preprocess_file result_file centroid_num boundary_factor sample_factor metric" << std::endl;
        exit(-1);
    }
    device_resources handle(std::getenv("GLIDE_DEVICE") ? std::atoi(std::getenv("GLIDE_DEVICE")) : 0);
    std::string data_file(argv[1]), preprocess_file(argv[2]), result_file(argv[3]);
    PartitionParameter param;
    param.centroid_num = std::stoi(argv[4]);
    param.boundary_factor = std::stof(argv[5]);
    param.sample_factor = std::stof(argv[6]);
    std::string metric(argv[7]);
    if (metric == "Euclidean") param.metric = Metric::Euclidean;
    else if (metric == "Cosine") param.metric = Metric::Cosine;

    std::ifstream probe(result_file);
    if (!probe.good()) {   // header as written by the reference (small_preprocess.cu:54-56)
        std::ofstream result_out(result_file, std::ios::app);
        result_out << "pre_time,knn_time,degree,index_time,beam,search_time,QPS,recall" << std::endl;
    }

    uint32_t file_dim = 0;   // rows are held padded to a multiple of four values (load.hpp); the files written below keep the data file's length
    auto h_data = load_point_data<float, uint32_t>(data_file, 4, &file_dim);
    const uint32_t num = h_data.extent(0), dim = h_data.extent(1);
    device_matrix<float, uint32_t> d_data(num, dim);
    copy_to_device(d_data.data_handle(), h_data.data_handle(), h_data.size());
    device_matrix<float> d_centroids(param.centroid_num, dim);
    host_vector<uint32_t> h_segment_start(param.centroid_num + 1), h_segment_length(param.centroid_num + 1);
    std::optional<device_matrix<float, uint32_t>> d_reorder_data;
    std::optional<device_vector<uint32_t>> d_map;

    preprocess<float, uint32_t>(handle, param, d_data.view(), d_reorder_data, d_map, h_segment_start.view(), h_segment_length.view(),
                                d_centroids.view(), result_file);

    host_matrix<float> h_centroids(param.centroid_num, dim);
    copy_to_host(h_centroids.data_handle(), d_centroids.data_handle(), h_centroids.size());
    host_matrix<float, uint32_t> h_reorder(d_reorder_data->extent(0), dim);
    copy_to_host(h_reorder.data_handle(), d_reorder_data->data_handle(), h_reorder.size());
    host_vector<uint32_t> h_map(d_map->size());
    copy_to_host(h_map.data_handle(), d_map->data_handle(), h_map.size());

    save_point_data<float, uint32_t>(preprocess_file + ".centroid", std::as_const(h_centroids).view(), file_dim);
    save_segment(preprocess_file + ".segment", std::as_const(h_segment_start).view(), std::as_const(h_segment_length).view());
    save_vector_data(preprocess_file + ".map", std::as_const(h_map).view());
    save_point_data<float, uint32_t>(preprocess_file + ".reorder", std::as_const(h_reorder).view(), file_dim);
    return 0;
}
