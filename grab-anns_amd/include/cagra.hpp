// Free functions of namespace cagra with the reference's signatures (src/index/cagra.cuh:44-147,
// src/index/cagra_opt.cuh) over the C ABI.  Device pointers in, device pointers out; errors become
// std::runtime_error, as the reference throws for a null graph (src/index/cagra.cu:858-860).
#pragma once
#include <cstdint>
#include <random>
#include <stdexcept>

#include "grab_anns.h"

namespace cagra {

constexpr int MAX_DEGREE = GRAB_MAX_DEGREE;  // src/index/cagra.cuh:24

struct BuildParams {  // src/index/cagra.cuh:30-33
    uint32_t intermediate_degree = 128;
    uint32_t graph_degree = 64;
};

struct SearchParams {  // src/index/cagra.cuh:35-42
    uint32_t itopk_size = 64;
    uint32_t search_width = 5;
    uint32_t min_iterations = 0;
    uint32_t max_iterations = 20;
    uint32_t hash_bitlen = 12;
    static constexpr uint32_t TEAM_SIZE = 32;
};

namespace detail {
inline void check(int rc) {
    if (rc != GRAB_OK) throw std::runtime_error(grab_last_error());
}
inline grab_search_params to_c(const SearchParams& p) {
    return grab_search_params{p.itopk_size, p.search_width, p.min_iterations, p.max_iterations, p.hash_bitlen};
}
// the reference seeds rand_xor_mask from std::random_device on every call (src/index/cagra.cu:885-886)
inline uint64_t random_mask() {
    std::random_device rd;
    return rd();
}
inline uint32_t next_power_of_2(uint32_t n) { return grab_next_power_of_2(n); }  // src/index/smem_cal.cuh:13-23
inline size_t calculate_and_check_smem(uint32_t itopk, uint32_t dim, uint32_t sw, uint32_t deg, uint32_t bitlen) {
    return grab_reference_smem_bytes(itopk, dim, sw, deg, bitlen);  // src/index/smem_cal.cuh:28-76
}
}  // namespace detail

// src/index/cagra.cu:69-210.  The reference writes the graph to HOST memory; so does this wrapper.
void generate_knn_graph(const float* d_dataset, size_t num_dataset, uint32_t dim, uint32_t k, uint32_t* h_knn_graph);

inline void optimize_prune_device(const uint32_t* d_knn, uint32_t* d_new, size_t n, uint32_t in_deg, uint32_t out_deg) {
    detail::check(grab_optimize_prune(d_knn, d_new, n, in_deg, out_deg, nullptr));
}

// src/index/cagra.cu:665-711: allocates *d_constructed_graph; the caller frees it with grab_device_free
inline void build(const float* d_dataset, size_t num_dataset, const uint32_t* d_raw_knn_graph, BuildParams params,
                  uint32_t** d_constructed_graph) {
    void* g = nullptr;
    detail::check(grab_device_malloc(&g, num_dataset * params.graph_degree * sizeof(uint32_t)));
    int rc = grab_build_graph(d_dataset, num_dataset, d_raw_knn_graph,
                              grab_build_params{params.intermediate_degree, params.graph_degree},
                              static_cast<uint32_t*>(g), nullptr);
    if (rc != GRAB_OK) {
        grab_device_free(g);
        detail::check(rc);
    }
    *d_constructed_graph = static_cast<uint32_t*>(g);
}

// src/index/cagra.cu:844-935
inline void search(const float* d_dataset, size_t num_dataset, uint32_t dim, const uint32_t* d_graph,
                   uint32_t graph_degree, const float* d_queries, int64_t num_queries, int64_t k, SearchParams params,
                   int64_t* d_out_indices, float* d_out_dists, const uint32_t* d_seeds = nullptr,
                   const uint32_t num_seeds = 0) {
    detail::check(grab_search(d_dataset, num_dataset, dim, d_graph, graph_degree, d_queries, num_queries, k,
                              detail::to_c(params), d_out_indices, d_out_dists, d_seeds, num_seeds,
                              detail::random_mask(), 0, nullptr));
}

// src/index/cagra_opt.cu:1108-1210
inline void search_opt(const float* d_dataset, uint32_t dim, size_t num_dataset, const uint32_t* d_graph,
                       uint32_t graph_degree, const float* d_queries, int64_t num_queries, int64_t k,
                       SearchParams params, int64_t* d_out_indices, float* d_out_dists, const uint32_t* d_seeds,
                       const uint32_t num_seeds_per_query, void* stream = nullptr) {
    detail::check(grab_search_opt(d_dataset, dim, num_dataset, d_graph, graph_degree, d_queries, num_queries, k,
                                  detail::to_c(params), d_out_indices, d_out_dists, d_seeds, num_seeds_per_query,
                                  detail::random_mask(), 0, stream));
}

// src/index/cagra_opt.cu:1212-1328
inline void search_bucket_opt(const float* d_dataset, uint32_t dim, size_t num_dataset, const uint32_t* d_graph,
                              uint32_t total_degree, uint32_t local_degree, const float* d_queries,
                              int64_t num_queries, int64_t k, SearchParams params, int64_t* d_out_indices,
                              float* d_out_dists, const uint32_t* d_seeds, const uint32_t num_seeds_per_query,
                              void* stream = nullptr) {
    detail::check(grab_search_bucket(d_dataset, dim, num_dataset, d_graph, total_degree, local_degree, d_queries,
                                     num_queries, k, detail::to_c(params), d_out_indices, d_out_dists, d_seeds,
                                     num_seeds_per_query, detail::random_mask(), 0, stream));
}

// src/index/cagra_opt.cu:1330-1442
inline void search_bucket_range(const float* d_dataset, uint32_t dim, size_t num_dataset, const uint32_t* d_graph,
                                uint64_t* d_ts, uint32_t total_degree, uint32_t local_degree, const float* d_queries,
                                int64_t num_queries, int64_t k, uint64_t start_bucket, uint64_t end_bucket,
                                SearchParams params, int64_t* d_out_indices, float* d_out_dists,
                                const uint32_t* d_seeds, const uint32_t num_seeds_per_query) {
    detail::check(grab_search_range(d_dataset, dim, num_dataset, d_graph, d_ts, total_degree, local_degree, d_queries,
                                    num_queries, k, start_bucket, end_bucket, detail::to_c(params), d_out_indices,
                                    d_out_dists, d_seeds, num_seeds_per_query, detail::random_mask(), 0, nullptr));
}

// src/index/cagra.cu:938-1015.  h_graph is unused by the reference's implementation and by this one.
inline void insert(const float* d_dataset, size_t num_existing, size_t num_new, const float* d_new_data,
                   uint32_t* d_graph, uint32_t* /*h_graph*/, uint32_t graph_degree, SearchParams search_params,
                   uint32_t dim) {
    uint64_t state = detail::random_mask() | (detail::random_mask() << 32);
    detail::check(grab_insert(d_dataset, dim, num_existing, num_new, d_new_data, d_graph, graph_degree,
                              detail::to_c(search_params), GRAB_METRIC_L2, &state, 0, 0, nullptr));
}

inline void generate_knn_graph(const float* d_dataset, size_t num_dataset, uint32_t dim, uint32_t k,
                               uint32_t* h_knn_graph) {
    void* d = nullptr;
    detail::check(grab_device_malloc(&d, num_dataset * k * sizeof(uint32_t)));
    int rc = grab_generate_knn_graph(d_dataset, num_dataset, dim, k, GRAB_METRIC_L2, static_cast<uint32_t*>(d), nullptr,
                                     nullptr);
    if (rc == GRAB_OK) rc = grab_copy_to_host(h_knn_graph, d, num_dataset * k * sizeof(uint32_t));
    grab_device_free(d);
    detail::check(rc);
}

}  // namespace cagra
