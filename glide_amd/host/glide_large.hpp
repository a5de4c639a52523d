// class GLIDE_large: data, graph and map live in pinned host memory; one partition at a time is staged through the
// GPU.  Reference: glide_large.cuh:14-212, glide_large_impl.cuh:14-507 (instantiated there for uint8 rows; uint8 or float here).
// On a GPU that holds the whole index (rows as fp32 + graph + map; 32 GB for 50M x 128) search() uploads it once and
// searches the partitions in place; the staged search is kept for indexes that do not fit.
// Partitions are independent on this path (no boundary list, no cross-partition merge), so build -> reverse edges ->
// refine run back to back on a staged partition instead of in three passes over the host arrays, and the copy of
// the next partition overlaps the kernels of the current one.
// build_with_merge (declared by the reference at glide_large.cuh:89-97, never defined there) is the large-path form of
// the small path's merge (glide_impl.cuh:77-256): the partitioning carries a boundary segment, the partitions' sub-graphs
// are placed into one graph that stays in device memory, the boundary copies join them, reverse edges are added.  The
// merged index is searched like a small index: rows and graph resident in HBM, one kernel, no staging per query batch.
#pragma once
#include <cfloat>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <optional>
#include <random>
#include <stdexcept>
#include <string>
#include <vector>

#include "load.hpp"
#include "mdarray.hpp"
#include "params.hpp"
#include "pinned.hpp"

namespace glide {

template <typename Data_t, typename Index_t>
class GLIDE_large {

public:
    // glide_large_impl.cuh:14-28: an index to be built
    GLIDE_large(device_resources& handle, uint32_t graph_degree, Metric metric, std::string& reorder_file, std::string& map_file,
                std::string& centroid_file, std::string& segment_file)
        : handle(handle), metric(metric), h_data(load_points_pinned<Data_t>(reorder_file)), h_map(load_vector_data(map_file)),
          h_centroids(load_point_data<float, uint32_t>(centroid_file, 16 / sizeof(Data_t))), h_segment_start(load_segment_start(segment_file)),
          h_segment_length(load_segment_length(segment_file)), h_start_point(h_segment_start.size()), h_graph(point_num(), graph_degree) {}
    // glide_large_impl.cuh:29-43: a finished index
    GLIDE_large(device_resources& handle, Metric metric, std::string& reorder_file, std::string& map_file, std::string& centroid_file,
                std::string& segment_file, std::string& start_point_file, std::string& graph_file)
        : handle(handle), metric(metric), h_data(load_points_pinned<Data_t>(reorder_file)), h_map(load_vector_data(map_file)),
          h_centroids(load_point_data<float, uint32_t>(centroid_file, 16 / sizeof(Data_t))), h_segment_start(load_segment_start(segment_file)),
          h_segment_length(load_segment_length(segment_file)), h_start_point(load_vector_data(start_point_file)),
          h_graph(load_matrix_pinned<uint32_t>(graph_file)) {}

    uint32_t dim() const { return h_data.extent(1); }
    Index_t num() const { return h_data.extent(0); }
    uint32_t graph_degree() const { return h_graph.extent(1); }
    uint32_t segment_num() const { return h_segment_start.size(); }
    uint32_t centroids_num() const { return h_centroids.extent(0); }
    // a partitioning made for a merged index has one segment more than centroids: the boundary copies, behind the points
    bool merged() const { return h_segment_start.size() == static_cast<size_t>(h_centroids.extent(0)) + 1; }
    Index_t point_num() const { return merged() ? h_segment_start.data_handle()[h_centroids.extent(0)] : h_data.extent(0); }
    const pinned_matrix<uint32_t>& graph_view() const { return h_graph; }
    host_vector_view<const uint32_t> start_point_view() const { return h_start_point.view(); }

    // glide_large_impl.cuh:328-345
    void build(IndexParameter& build_param, SearchParameter& search_param_knn, SearchParameter& search_param_refine,
               const pinned_matrix<uint32_t>& h_knn_graph, std::string& result_file) {
        std::mt19937 generator(build_param.seed);   // start_point_select (glide_large_impl.cuh:55-76)
        for (uint32_t i = 0; i < segment_num(); i++) {
            const uint32_t len = h_segment_length(i);
            h_start_point(i) = len ? std::uniform_int_distribution<uint32_t>(0, len - 1)(generator) : 0;
        }
        const uint32_t knn_degree = h_knn_graph.extent(1), deg = graph_degree();
        uint32_t max_len = 0;
        for (uint32_t s = 0; s < segment_num(); s++) max_len = std::max(max_len, h_segment_length(s));
        staged_rows<Data_t> d_data[2] = {staged_rows<Data_t>(max_len, dim()), staged_rows<Data_t>(max_len, dim())};
        device_matrix<uint32_t> d_knn[2] = {device_matrix<uint32_t>(max_len, knn_degree), device_matrix<uint32_t>(max_len, knn_degree)};
        device_matrix<uint32_t> d_graph(max_len, deg), d_rev(max_len, deg);
        device_vector<uint32_t> d_rev_count(max_len);
        const size_t wb = glide_hip_reverse_edges_workspace_bytes(max_len, deg);
        device_buffer ws(wb);
        const int mc = metric_code(metric);
        stager st;
        auto stage = [&](uint32_t s) {
            const int b = s & 1;
            const size_t start = h_segment_start(s), len = h_segment_length(s);
            st.before_copy(b);
            d_data[b].upload_async(h_data.row(start), len, st.copy_stream());
            hip_try(glide_hip_memcpy_h2d_async(d_knn[b].data_handle(), h_knn_graph.row(start), len * knn_degree * sizeof(uint32_t), st.copy_stream()), "h2d knn");
            st.after_copy(b);
        };
        void* t0 = nullptr;
        void* t1 = nullptr;
        hip_try(glide_hip_event_create(&t0), "glide_hip_event_create");
        hip_try(glide_hip_event_create(&t1), "glide_hip_event_create");
        void* cs = st.compute_stream();
        hip_try(glide_hip_event_record(t0, cs), "glide_hip_event_record");
        if (segment_num()) stage(0);
        for (uint32_t s = 0; s < segment_num(); s++) {
            const int b = s & 1;
            const uint32_t len = h_segment_length(s);
            if (s + 1 < segment_num()) stage(s + 1);
            st.before_compute(b);
            d_data[b].widen(len, cs);
            SearchParameter& p = search_param_knn;
            hip_try(glide_hip_build_segment(d_data[b].data_handle(), len, dim(), d_knn[b].data_handle(), knn_degree, h_start_point(s), deg, p.beam,
                                            p.max_iterations, p.min_iterations, p.hash_bit, p.hash_reset_interval, build_param.relaxant_factor, mc,
                                            d_graph.data_handle(), nullptr, cs),
                    "glide_hip_build_segment");
            hip_try(glide_hip_reverse_edges(d_graph.data_handle(), len, deg, d_rev.data_handle(), d_rev_count.data_handle(), ws.get(), wb, cs),
                    "glide_hip_reverse_edges");
            hip_try(glide_hip_insert_reverse(d_graph.data_handle(), d_rev.data_handle(), d_rev_count.data_handle(), len, deg, cs),
                    "glide_hip_insert_reverse");
            const uint32_t* result = d_graph.data_handle();
            if (search_param_refine.beam != 0) {
                SearchParameter& r = search_param_refine;
                hip_try(glide_hip_refine_segment(d_data[b].data_handle(), len, dim(), d_graph.data_handle(), d_rev.data_handle(), deg, h_start_point(s),
                                                 r.beam, r.max_iterations, r.min_iterations, r.hash_bit, r.hash_reset_interval,
                                                 build_param.relaxant_factor, mc, nullptr, cs),
                        "glide_hip_refine_segment");
                result = d_rev.data_handle();
            }
            hip_try(glide_hip_memcpy_d2h_async(h_graph.row(h_segment_start(s)), result, static_cast<size_t>(len) * deg * sizeof(uint32_t), cs), "d2h graph");
            st.after_compute(b);
        }
        hip_try(glide_hip_event_record(t1, cs), "glide_hip_event_record");
        st.sync();
        float ms = 0.f;
        hip_try(glide_hip_event_elapsed_ms(t0, t1, &ms), "glide_hip_event_elapsed_ms");
        glide_hip_event_destroy(t0);
        glide_hip_event_destroy(t1);
        const float build_time = ms / 1000.0f;
        std::cout << "index build time: " << build_time << " s" << std::endl;
        std::ofstream result_out(result_file, std::ios::app);
        result_out << build_time << ",";
    }

    // Declared at glide_large.cuh:89-97.  Sub-graphs per staged partition as in build(); rows are placed into the merged
    // graph (device memory, reorder-id space); the boundary segment is built the same way and merged into the rows of
    // the points its copies duplicate (map_to_graph_boundary, graph_kernel.cuh:160-247); reverse edges over the whole
    // graph (glide_impl.cuh:194-256).  No refinement pass: the declaration takes no refine parameter.
    void build_with_merge(IndexParameter& build_param, SearchParameter& search_param_knn, const pinned_matrix<uint32_t>& h_knn_graph,
                          std::string& result_file) {
        SearchParameter no_refine;
        no_refine.beam = 0;
        build_with_merge(build_param, search_param_knn, no_refine, h_knn_graph, result_file);
    }

    // The same with the small path's last stage (refine_kernel, glide_impl.cuh:258-316) when search_param_refine.beam != 0:
    // all rows are then uploaded next to the merged graph (50M x 128 fp32 = 25.6 GB of the 288 GB) and rows with empty
    // slots are completed by a search over the whole graph.
    void build_with_merge(IndexParameter& build_param, SearchParameter& search_param_knn, SearchParameter& search_param_refine,
                          const pinned_matrix<uint32_t>& h_knn_graph, std::string& result_file) {
        if (!merged()) throw std::invalid_argument("build_with_merge: the partitioning has no boundary segment");
        std::mt19937 generator(build_param.seed);
        for (uint32_t i = 0; i < segment_num(); i++) {
            const uint32_t len = h_segment_length(i);
            h_start_point(i) = len ? std::uniform_int_distribution<uint32_t>(0, len - 1)(generator) : 0;
        }
        const uint32_t knn_degree = h_knn_graph.extent(1), deg = graph_degree(), c = centroids_num();
        const uint32_t n = point_num(), copies = h_segment_length(c);
        // home row of every boundary copy: the reorder row of the point it duplicates
        std::vector<uint32_t> home(copies);
        {
            std::vector<uint32_t> row_of(n);
            for (uint32_t r = 0; r < n; r++) row_of[h_map(r)] = r;
            for (uint32_t i = 0; i < copies; i++) home[i] = row_of[h_map(n + i)];
        }
        uint32_t max_len = 0;
        for (uint32_t s = 0; s < segment_num(); s++) max_len = std::max(max_len, h_segment_length(s));
        staged_rows<Data_t> d_data[2] = {staged_rows<Data_t>(max_len, dim()), staged_rows<Data_t>(max_len, dim())};
        device_matrix<uint32_t> d_knn[2] = {device_matrix<uint32_t>(max_len, knn_degree), device_matrix<uint32_t>(max_len, knn_degree)};
        device_matrix<uint32_t> d_local(max_len, deg), d_merged(n, deg), d_rev(n, deg);
        device_vector<uint32_t> d_rev_count(n), d_home(copies ? copies : 1);
        if (copies) copy_to_device(d_home.data_handle(), home.data(), copies);
        const size_t wb = glide_hip_reverse_edges_workspace_bytes(n, deg);
        device_buffer ws(wb);
        const int mc = metric_code(metric);
        stager st;
        auto stage = [&](uint32_t s) {
            const int b = s & 1;
            const size_t start = h_segment_start(s), len = h_segment_length(s);
            st.before_copy(b);
            d_data[b].upload_async(h_data.row(start), len, st.copy_stream());
            hip_try(glide_hip_memcpy_h2d_async(d_knn[b].data_handle(), h_knn_graph.row(start), len * knn_degree * sizeof(uint32_t), st.copy_stream()), "h2d knn");
            st.after_copy(b);
        };
        void* t0 = nullptr;
        void* t1 = nullptr;
        hip_try(glide_hip_event_create(&t0), "glide_hip_event_create");
        hip_try(glide_hip_event_create(&t1), "glide_hip_event_create");
        void* cs = st.compute_stream();
        hip_try(glide_hip_event_record(t0, cs), "glide_hip_event_record");
        hip_try(glide_hip_fill_u32(d_merged.data_handle(), 0xffffffffu, d_merged.size(), cs), "glide_hip_fill_u32");
        stage(0);
        for (uint32_t s = 0; s < segment_num(); s++) {
            const int b = s & 1;
            const uint32_t len = h_segment_length(s);
            if (s + 1 < segment_num()) stage(s + 1);
            st.before_compute(b);
            d_data[b].widen(len, cs);
            SearchParameter& p = search_param_knn;
            hip_try(glide_hip_build_segment(d_data[b].data_handle(), len, dim(), d_knn[b].data_handle(), knn_degree, h_start_point(s), deg, p.beam,
                                            p.max_iterations, p.min_iterations, p.hash_bit, p.hash_reset_interval, build_param.relaxant_factor, mc,
                                            d_local.data_handle(), nullptr, cs),
                    "glide_hip_build_segment");
            if (s < c)
                hip_try(glide_hip_place_segment_graph(d_local.data_handle(), len, deg, h_segment_start(s), d_merged.data_handle(), cs),
                        "glide_hip_place_segment_graph");
            else   // the boundary segment is the last one: every partition's rows are in place by now
                hip_try(glide_hip_merge_boundary_graph(d_local.data_handle(), len, deg, d_home.data_handle(), d_merged.data_handle(), cs),
                        "glide_hip_merge_boundary_graph");
            st.after_compute(b);
        }
        hip_try(glide_hip_reverse_edges(d_merged.data_handle(), n, deg, d_rev.data_handle(), d_rev_count.data_handle(), ws.get(), wb, cs),
                "glide_hip_reverse_edges");
        hip_try(glide_hip_insert_reverse(d_merged.data_handle(), d_rev.data_handle(), d_rev_count.data_handle(), n, deg, cs), "glide_hip_insert_reverse");
        const uint32_t* result = d_merged.data_handle();
        std::optional<device_matrix<float>> d_rows, d_centroids;
        std::optional<device_vector<uint32_t>> d_entries;
        std::optional<staged_rows<Data_t>> slot;
        if (search_param_refine.beam != 0) {
            SearchParameter& r = search_param_refine;
            d_rows.emplace(n, dim());
            slot.emplace(sizeof(Data_t) == 1 ? upload_piece(n) : 1, dim());
            upload_rows(d_rows->data_handle(), *slot, cs);
            d_centroids.emplace(c, dim());
            d_entries.emplace(c);
            std::vector<uint32_t> entry(c);
            for (uint32_t s = 0; s < c; s++) entry[s] = h_segment_start(s) + h_start_point(s);
            hip_try(glide_hip_memcpy_h2d(d_centroids->data_handle(), h_centroids.data_handle(), h_centroids.size() * sizeof(float), cs), "h2d centroids");
            hip_try(glide_hip_memcpy_h2d(d_entries->data_handle(), entry.data(), c * sizeof(uint32_t), cs), "h2d entries");
            hip_try(glide_hip_refine_merged(d_rows->data_handle(), n, dim(), d_merged.data_handle(), d_rev.data_handle(), deg,
                                            d_centroids->data_handle(), c, d_entries->data_handle(), r.beam, r.max_iterations, r.min_iterations,
                                            r.hash_bit, r.hash_reset_interval, build_param.relaxant_factor, mc, nullptr, nullptr, cs),
                    "glide_hip_refine_merged");
            result = d_rev.data_handle();
        }
        hip_try(glide_hip_memcpy_d2h_async(h_graph.data_handle(), result, d_merged.size() * sizeof(uint32_t), cs), "d2h graph");
        hip_try(glide_hip_event_record(t1, cs), "glide_hip_event_record");
        st.sync();
        float ms = 0.f;
        hip_try(glide_hip_event_elapsed_ms(t0, t1, &ms), "glide_hip_event_elapsed_ms");
        glide_hip_event_destroy(t0);
        glide_hip_event_destroy(t1);
        const float build_time = ms / 1000.0f;
        std::cout << "index build time: " << build_time << " s" << std::endl;
        std::ofstream result_out(result_file, std::ios::app);
        result_out << build_time << ",";
    }

    // glide_large_impl.cuh:347-507
    void search(SearchParameter& param, uint32_t min_segment_num, float boundary_factor, device_matrix_view<Data_t> d_query_view,
                host_matrix_view<uint32_t> h_result_ids_view, host_matrix_view<float> h_result_distances_view, std::string& result_file) {
        if (merged()) {
            search_merged(param, d_query_view, h_result_ids_view, h_result_distances_view, result_file);
            return;
        }
        // 288 GB of HBM hold what the reference has to stage for every query batch (50M x 128 fp32 rows + graph = 32 GB):
        // when the whole index fits it is uploaded once and the partitions are searched in place; the staged path below
        // remains for indexes that do not fit (or when GLIDE_LARGE_STAGED is set).
        if (!std::getenv("GLIDE_LARGE_STAGED") && !resident_failed) {
            bool first_use = false;
            try {
                first_use = make_resident();
            } catch (const hip_error&) {
                r_data.reset(); r_graph.reset(); r_centroids.reset(); r_start_points.reset(); r_map.reset();
                r_segment_starts.reset(); r_local_start_points.reset();
                resident_failed = true;
            }
            if (!resident_failed) {
                search_resident(param, min_segment_num, boundary_factor, d_query_view, h_result_ids_view, h_result_distances_view, result_file, first_use);
                return;
            }
        }
        const uint32_t query_number = d_query_view.extent(0), top_k = param.top_k, deg = graph_degree(), c = centroids_num();
        device_matrix<uint32_t> d_final_ids(query_number, top_k), d_segment_ids(query_number, c);
        device_matrix<float> d_final_dists(query_number, top_k), d_centroids(c, dim());
        copy_to_device(d_centroids.data_handle(), h_centroids.data_handle(), h_centroids.size());
        uint32_t max_len = 0;
        for (uint32_t s = 0; s < segment_num(); s++) max_len = std::max(max_len, h_segment_length(s));
        staged_rows<Data_t> d_data[2] = {staged_rows<Data_t>(max_len, dim()), staged_rows<Data_t>(max_len, dim())};
        device_matrix<uint32_t> d_graph[2] = {device_matrix<uint32_t>(max_len, deg), device_matrix<uint32_t>(max_len, deg)};
        device_vector<uint32_t> d_map[2] = {device_vector<uint32_t>(max_len), device_vector<uint32_t>(max_len)};
        const int mc = metric_code(metric);
        stager st;
        void* cs = st.compute_stream();
        auto stage = [&](uint32_t s) {
            const int b = s & 1;
            const size_t start = h_segment_start(s), len = h_segment_length(s);
            st.before_copy(b);
            d_data[b].upload_async(h_data.row(start), len, st.copy_stream());
            hip_try(glide_hip_memcpy_h2d_async(d_graph[b].data_handle(), h_graph.row(start), len * deg * sizeof(uint32_t), st.copy_stream()), "h2d graph");
            hip_try(glide_hip_memcpy_h2d_async(d_map[b].data_handle(), h_map.data_handle() + start, len * sizeof(uint32_t), st.copy_stream()), "h2d map");
            st.after_copy(b);
        };
        void* t0 = nullptr;
        void* t1 = nullptr;
        hip_try(glide_hip_event_create(&t0), "glide_hip_event_create");
        hip_try(glide_hip_event_create(&t1), "glide_hip_event_create");
        hip_try(glide_hip_fill_u32(d_final_ids.data_handle(), 0xffffffffu, d_final_ids.size(), cs), "glide_hip_fill_u32");
        const float fmax = FLT_MAX;
        uint32_t fmax_bits;
        std::memcpy(&fmax_bits, &fmax, 4);
        hip_try(glide_hip_fill_u32(reinterpret_cast<uint32_t*>(d_final_dists.data_handle()), fmax_bits, d_final_dists.size(), cs), "glide_hip_fill_u32");
        hip_try(glide_hip_event_record(t0, cs), "glide_hip_event_record");
        // uint8 queries (large_search.cu:111) are widened once; every kernel below reads fp32 queries
        device_matrix<float> d_query_f32(sizeof(Data_t) == 1 ? query_number : 0, dim());
        const float* d_queries = reinterpret_cast<const float*>(d_query_view.data_handle());
        if (sizeof(Data_t) == 1) {
            hip_try(glide_hip_widen_u8(reinterpret_cast<const unsigned char*>(d_query_view.data_handle()), static_cast<size_t>(query_number) * dim(),
                                       d_query_f32.data_handle(), cs),
                    "glide_hip_widen_u8");
            d_queries = d_query_f32.data_handle();
        }
        hip_try(glide_hip_select_segments(d_queries, query_number, dim(), d_centroids.data_handle(), c, min_segment_num,
                                          boundary_factor, mc, d_segment_ids.data_handle(), cs),
                "glide_hip_select_segments");
        if (segment_num()) stage(0);
        for (uint32_t s = 0; s < segment_num(); s++) {
            const int b = s & 1;
            if (s + 1 < segment_num()) stage(s + 1);
            st.before_compute(b);
            d_data[b].widen(h_segment_length(s), cs);
            hip_try(glide_hip_search_sub(d_data[b].data_handle(), dim(), d_graph[b].data_handle(), deg, d_map[b].data_handle(),
                                         d_queries, query_number, d_segment_ids.data_handle(), c, s, h_start_point(s), top_k,
                                         param.beam, param.max_iterations, param.min_iterations, param.hash_bit, param.hash_reset_interval, mc,
                                         d_final_ids.data_handle(), d_final_dists.data_handle(), nullptr, cs),
                    "glide_hip_search_sub");
            st.after_compute(b);
        }
        hip_try(glide_hip_event_record(t1, cs), "glide_hip_event_record");
        st.sync();
        float ms = 0.f;
        hip_try(glide_hip_event_elapsed_ms(t0, t1, &ms), "glide_hip_event_elapsed_ms");
        glide_hip_event_destroy(t0);
        glide_hip_event_destroy(t1);
        const float search_time = ms / 1000.0f;   // staging included: this is what a caller of the host-resident index sees
        std::cout << "query time: " << search_time << " s" << "   " << "QPS: " << static_cast<float>(query_number) / search_time << std::endl;
        std::ofstream result;
        result.setf(std::ios::fixed);
        result.open(result_file, std::ios::app);
        result << search_time << "," << static_cast<float>(query_number) / search_time << ",";
        result.close();
        copy_to_host(h_result_ids_view.data_handle(), d_final_ids.data_handle(), d_final_ids.size());
        copy_to_host(h_result_distances_view.data_handle(), d_final_dists.data_handle(), d_final_dists.size());
    }

    // Search of a merged index: the rows (widened to fp32) and the graph are uploaded once and stay in device memory; a
    // query batch is one launch of the small path's search kernel with every centroid ranked for the entry point.
    // Result ids are input row numbers (through the map), as from the staged search.
    void search_merged(SearchParameter& param, device_matrix_view<Data_t> d_query_view, host_matrix_view<uint32_t> h_result_ids_view,
                       host_matrix_view<float> h_result_distances_view, std::string& result_file) {
        const uint32_t query_number = d_query_view.extent(0), top_k = param.top_k, deg = graph_degree(), c = centroids_num(), n = point_num();
        const bool first_use = make_resident();
        device_matrix<uint32_t> d_ids(query_number, top_k);
        device_matrix<float> d_dists(query_number, top_k);
        device_matrix<float> d_query_f32(sizeof(Data_t) == 1 ? query_number : 0, dim());
        const float* d_queries = reinterpret_cast<const float*>(d_query_view.data_handle());
        if (first_use && query_number && !std::getenv("GLIDE_COLD_SEARCH"))   // part of bringing the index up: the first launch of a kernel loads its code
            hip_try(glide_hip_search_merged(r_data->data_handle(), n, dim(), r_graph->data_handle(), deg, r_centroids->data_handle(), c,
                                            r_start_points->data_handle(), r_data->data_handle(), 1, top_k, param.beam, param.max_iterations,
                                            param.min_iterations, param.hash_bit, param.hash_reset_interval, metric_code(metric),
                                            d_ids.data_handle(), d_dists.data_handle(), nullptr, handle.stream()),
                    "glide_hip_search_merged");
        gpu_timer timer;
        timer.start();
        if (sizeof(Data_t) == 1) {
            hip_try(glide_hip_widen_u8(reinterpret_cast<const unsigned char*>(d_query_view.data_handle()), static_cast<size_t>(query_number) * dim(),
                                       d_query_f32.data_handle(), handle.stream()),
                    "glide_hip_widen_u8");
            d_queries = d_query_f32.data_handle();
        }
        hip_try(glide_hip_search_merged(r_data->data_handle(), n, dim(), r_graph->data_handle(), deg, r_centroids->data_handle(), c,
                                        r_start_points->data_handle(), d_queries, query_number, top_k, param.beam, param.max_iterations,
                                        param.min_iterations, param.hash_bit, param.hash_reset_interval, metric_code(metric), d_ids.data_handle(),
                                        d_dists.data_handle(), nullptr, handle.stream()),
                "glide_hip_search_merged");
        const float search_time = timer.stop();
        std::cout << "query time: " << search_time << " s" << "   " << "QPS: " << static_cast<float>(query_number) / search_time << std::endl;
        if (std::getenv("GLIDE_SEARCH_COUNTERS") && query_number) {
            // the same launch once more, untimed, with the kernel's own tallies (what its algorithmic traffic is computed from)
            device_buffer d_counters(GLIDE_COUNTER_STRIPES * 3 * sizeof(unsigned long long));
            hip_try(glide_hip_fill_u32(static_cast<uint32_t*>(d_counters.get()), 0u, GLIDE_COUNTER_STRIPES * 6, handle.stream()), "glide_hip_fill_u32");
            hip_try(glide_hip_search_merged(r_data->data_handle(), n, dim(), r_graph->data_handle(), deg, r_centroids->data_handle(), c,
                                            r_start_points->data_handle(), d_queries, query_number, top_k, param.beam, param.max_iterations,
                                            param.min_iterations, param.hash_bit, param.hash_reset_interval, metric_code(metric), d_ids.data_handle(),
                                            d_dists.data_handle(), static_cast<unsigned long long*>(d_counters.get()), handle.stream()),
                    "glide_hip_search_merged");
            std::vector<unsigned long long> h(GLIDE_COUNTER_STRIPES * 3);
            copy_to_host(h.data(), static_cast<unsigned long long*>(d_counters.get()), h.size());
            unsigned long long sum[3] = {0, 0, 0};
            for (size_t i = 0; i < h.size(); i++) sum[i % 3] += h[i];
            std::cout << "search counters: iterations " << sum[0] << " rows " << sum[1] << " graph_rows " << sum[2] << std::endl;
        }
        std::ofstream result;
        result.setf(std::ios::fixed);
        result.open(result_file, std::ios::app);
        result << search_time << "," << static_cast<float>(query_number) / search_time << ",";
        result.close();
        copy_to_host(h_result_ids_view.data_handle(), d_ids.data_handle(), d_ids.size());
        copy_to_host(h_result_distances_view.data_handle(), d_dists.data_handle(), d_dists.size());
        for (size_t i = 0; i < h_result_ids_view.size(); i++) {
            uint32_t& id = h_result_ids_view.data_handle()[i];
            if (id < n) id = h_map(id);
        }
    }

    // The per-partition search of glide_large_impl.cuh:347-507 on an index that is resident in device memory: the same
    // searches and the same order of result merges as the staged path, without the copies and in three launches
    // (queries grouped by partition, one wavefront per query and selected partition, one merge per query).
    void search_resident(SearchParameter& param, uint32_t min_segment_num, float boundary_factor, device_matrix_view<Data_t> d_query_view,
                         host_matrix_view<uint32_t> h_result_ids_view, host_matrix_view<float> h_result_distances_view, std::string& result_file,
                         bool first_use) {
        const uint32_t query_number = d_query_view.extent(0), top_k = param.top_k, deg = graph_degree(), c = centroids_num();
        device_matrix<uint32_t> d_final_ids(query_number, top_k), d_segment_ids(query_number, c);
        device_matrix<float> d_final_dists(query_number, top_k);
        device_matrix<float> d_query_f32(sizeof(Data_t) == 1 ? query_number : 0, dim());
        const size_t swb = glide_hip_search_partitions_workspace_bytes(query_number, c, top_k);
        device_buffer search_ws(swb);
        const int mc = metric_code(metric);
        void* cs = handle.stream();
        auto run = [&](uint32_t queries) {
            const float* d_queries = reinterpret_cast<const float*>(d_query_view.data_handle());
            if (sizeof(Data_t) == 1) {
                hip_try(glide_hip_widen_u8(reinterpret_cast<const unsigned char*>(d_query_view.data_handle()), static_cast<size_t>(queries) * dim(),
                                           d_query_f32.data_handle(), cs),
                        "glide_hip_widen_u8");
                d_queries = d_query_f32.data_handle();
            }
            hip_try(glide_hip_select_segments(d_queries, queries, dim(), r_centroids->data_handle(), c, min_segment_num, boundary_factor, mc,
                                              d_segment_ids.data_handle(), cs),
                    "glide_hip_select_segments");
            // one wavefront per (query, selected partition), the heads merged per query in partition order
            hip_try(glide_hip_search_partitions(r_data->data_handle(), dim(), r_graph->data_handle(), deg, r_map->data_handle(),
                                                r_segment_starts->data_handle(), r_local_start_points->data_handle(), c, d_queries, queries,
                                                d_segment_ids.data_handle(), top_k, param.beam, param.max_iterations, param.min_iterations,
                                                param.hash_bit, param.hash_reset_interval, mc, d_final_ids.data_handle(),
                                                d_final_dists.data_handle(), search_ws.get(), swb, nullptr, cs),
                    "glide_hip_search_partitions");
        };
        if (first_use && query_number && !std::getenv("GLIDE_COLD_SEARCH")) run(1);   // part of bringing the index up: the first launch of a kernel loads its code
        gpu_timer timer;
        timer.start();
        run(query_number);
        const float search_time = timer.stop();
        std::cout << "query time: " << search_time << " s" << "   " << "QPS: " << static_cast<float>(query_number) / search_time << std::endl;
        std::ofstream result;
        result.setf(std::ios::fixed);
        result.open(result_file, std::ios::app);
        result << search_time << "," << static_cast<float>(query_number) / search_time << ",";
        result.close();
        copy_to_host(h_result_ids_view.data_handle(), d_final_ids.data_handle(), d_final_ids.size());
        copy_to_host(h_result_distances_view.data_handle(), d_final_dists.data_handle(), d_final_dists.size());
    }

private:
    static uint32_t upload_piece(uint32_t n) { return std::min<uint32_t>(n, 1u << 20); }

    // rows [0, point_num()) to device memory as fp32, in stream order (uint8 rows cross PCIe as bytes, one piece at a
    // time through `slot`, and are widened on the GPU)
    void upload_rows(float* dst_rows, staged_rows<Data_t>& slot, void* stream) {
        const uint32_t n = point_num(), piece = upload_piece(n);
        for (uint32_t first = 0; first < n; first += piece) {
            const uint32_t count = std::min(piece, n - first);
            float* dst = dst_rows + static_cast<size_t>(first) * dim();
            if (sizeof(Data_t) == 1) {
                slot.upload_async(h_data.row(first), count, stream);
                hip_try(glide_hip_widen_u8(reinterpret_cast<const unsigned char*>(slot.stored()), static_cast<size_t>(count) * dim(), dst, stream),
                        "glide_hip_widen_u8");
            } else {
                hip_try(glide_hip_memcpy_h2d_async(dst, h_data.row(first), static_cast<size_t>(count) * dim() * sizeof(float), stream),
                        "glide_hip_memcpy_h2d_async");
            }
        }
    }

    // one-time upload of the index (rows as fp32, graph, centroids, entry points, and the map for the per-partition search)
    bool make_resident() {
        if (r_data) return false;
        const uint32_t n = point_num(), c = centroids_num(), deg = graph_degree();
        gpu_timer timer;
        timer.start();
        r_data.emplace(n, dim());
        {
            staged_rows<Data_t> slot(sizeof(Data_t) == 1 ? upload_piece(n) : 1, dim());
            upload_rows(r_data->data_handle(), slot, handle.stream());
            handle.sync();
        }
        r_graph.emplace(n, deg);
        copy_to_device(r_graph->data_handle(), h_graph.data_handle(), h_graph.size());
        r_centroids.emplace(c, dim());
        copy_to_device(r_centroids->data_handle(), h_centroids.data_handle(), h_centroids.size());
        std::vector<uint32_t> entry(c);
        for (uint32_t s = 0; s < c; s++) entry[s] = h_segment_start(s) + h_start_point(s);
        r_start_points.emplace(c);
        copy_to_device(r_start_points->data_handle(), entry.data(), c);
        if (!merged()) {   // the per-partition search writes input row numbers itself and addresses the partitions on the device
            r_map.emplace(n);
            copy_to_device(r_map->data_handle(), h_map.data_handle(), n);
            r_segment_starts.emplace(c);
            copy_to_device(r_segment_starts->data_handle(), h_segment_start.data_handle(), c);
            std::vector<uint32_t> local(c);
            for (uint32_t s = 0; s < c; s++) local[s] = h_segment_length(s) ? h_start_point(s) : 0xffffffffu;   // empty partitions are skipped
            r_local_start_points.emplace(c);
            copy_to_device(r_local_start_points->data_handle(), local.data(), c);
        }
        std::cout << "index upload time: " << timer.stop() << " s" << std::endl;
        return true;
    }

    std::optional<device_matrix<float>> r_data;
    std::optional<device_matrix<uint32_t>> r_graph;
    std::optional<device_matrix<float>> r_centroids;
    std::optional<device_vector<uint32_t>> r_start_points, r_map, r_segment_starts, r_local_start_points;
    bool resident_failed = false;
    device_resources& handle;
    Metric metric;
    pinned_matrix<Data_t> h_data;
    host_vector<uint32_t> h_map;
    host_matrix<float> h_centroids;
    host_vector<uint32_t> h_segment_start, h_segment_length, h_start_point;
    pinned_matrix<uint32_t> h_graph;
};

}  // namespace glide
