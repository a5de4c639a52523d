// Parameter structs and derived-size arithmetic, as in the reference's params.cuh:5-99.
#pragma once
#include <algorithm>
#include <cstdint>

namespace glide {

enum class Metric { Euclidean, Cosine };   // params.cuh:5-8

struct PartitionParameter {                // params.cuh:10-15
    uint32_t centroid_num = 10;
    float boundary_factor = 1.05f;
    float sample_factor = 0.01f;
    Metric metric = Metric::Euclidean;
    uint32_t kmeans_iterations = 20;       // Lloyd steps replacing cuvs::cluster::kmeans::fit
    uint32_t seed = 7;                     // the reference shuffles with std::random_device
};

struct NNDescentParameter {                // params.cuh:17-25
    uint32_t graph_degree = 64;
    uint32_t intermediate_graph_degree = 128;
    uint32_t max_iterations = 20;
    float termination_threshold = 0.0001f;
    uint32_t seed = 0;
    explicit NNDescentParameter(size_t degree) : graph_degree(degree), intermediate_graph_degree(1.5 * degree) {}
};

struct IndexParameter {                    // params.cuh:27-35
    uint32_t graph_degree = 32;
    uint32_t knn_degree = 32;
    float relaxant_factor = 1.05f;
    Metric metric = Metric::Euclidean;
    uint32_t seed = 11;                    // start-point selection (std::random_device in the reference)
};

struct SearchParameter {                   // params.cuh:37-47
    uint32_t top_k = 10;
    uint32_t beam = 100;
    uint32_t max_iterations = 0;
    uint32_t min_iterations = 0;
    uint32_t hash_bit = 0;
    float hash_max_fill_rate = 0.5f;
    uint32_t hashmap_min_bitlen = 0;
    uint32_t hash_reset_interval = 1;
    uint32_t search_block_size = 0;
};

inline uint32_t hashmap_size(uint32_t bitlen) { return 1u << bitlen; }   // hashmap.cuh:23

inline uint32_t calculate_hash_bitlen(uint32_t beam, uint32_t graph_degree, float hashmap_max_fill_rate, uint32_t hashmap_min_bitlen) {
    uint32_t max_visited_nodes = beam + graph_degree;   // params.cuh:49-66
    uint32_t min_bitlen = 8, max_bitlen = 13;
    if (min_bitlen < hashmap_min_bitlen) min_bitlen = hashmap_min_bitlen;
    uint32_t hash_bitlen = min_bitlen;
    while (max_visited_nodes > hashmap_size(hash_bitlen) * hashmap_max_fill_rate) hash_bitlen += 1;
    if (hash_bitlen > max_bitlen) hash_bitlen = max_bitlen;
    return hash_bitlen;
}

inline uint32_t calculate_hash_reset_interval(uint32_t beam, uint32_t graph_degree, float hashmap_max_fill_rate, uint32_t hash_bitlen) {
    uint32_t hash_reset_interval = 1;                    // params.cuh:68-80
    while (true) {
        const auto max_visited_nodes = beam + graph_degree * (hash_reset_interval + 1);
        if (max_visited_nodes > hashmap_size(hash_bitlen) * hashmap_max_fill_rate) break;
        hash_reset_interval += 1;
    }
    return hash_reset_interval;
}

inline void adjust_search_params(uint32_t min_iterations, uint32_t& max_iterations, uint32_t& beam) {   // params.cuh:82-99
    uint32_t m = max_iterations;
    if (max_iterations == 0) m = 1 + std::min(beam * 1.1, beam + 10.0);
    if (max_iterations < min_iterations) m = min_iterations;
    if (max_iterations < m) max_iterations = m;
    if (beam % 32) beam += 32 - (beam % 32);
}

inline int metric_code(Metric m) { return m == Metric::Euclidean ? 0 : 1; }

}  // namespace glide
