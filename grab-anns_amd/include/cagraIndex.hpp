// cagra::CagraIndex with the reference's public surface (src/cagraIndex.hpp:12-119) as a header-only
// shell over the C ABI: same method names, argument meaning and error behaviour (std::runtime_error;
// silent return on an empty index).  Non-copyable, like the reference (unique_ptr members).
#pragma once
#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

#include "cagra.hpp"
#include "grab_anns.h"

namespace cagra {

class CagraIndex {
public:
    CagraIndex(uint32_t dim, uint32_t graph_degree = 64, size_t vmm_max_bytes = 20ULL * 1024 * 1024 * 1024) {
        detail::check(grab_index_create(dim, graph_degree, 0, vmm_max_bytes, &h_));
    }
    ~CagraIndex() { grab_index_destroy(h_); }
    CagraIndex(const CagraIndex&) = delete;
    CagraIndex& operator=(const CagraIndex&) = delete;

    void add(size_t num_vectors, const float* add_vectors, const uint64_t* add_timestamps = nullptr) {
        detail::check(grab_index_add(h_, num_vectors, add_vectors, add_timestamps));
    }
    void build() { detail::check(grab_index_build(h_)); }
    void insert(size_t new_vectors, const float* insert_vectors, const uint64_t* insert_timestamps = nullptr) {
        detail::check(grab_index_insert(h_, new_vectors, insert_vectors, insert_timestamps));
    }
    void query(const float* host_queries, size_t num_queries, int k, int64_t* host_indices, float* host_dists,
               uint32_t* seeds = nullptr, size_t num_seeds_per_query = 0) {
        detail::check(grab_index_search(h_, host_queries, num_queries, k, host_indices, host_dists, seeds, num_seeds_per_query));
    }
    // [start_ts, end_ts); range_radius >= 0.99 searches unfiltered (src/cagraIndex.cu:305,323)
    void query_range(const float* host_queries, size_t num_queries, int k, float range_radius, uint64_t start_ts,
                     uint64_t end_ts, int64_t* host_indices, float* host_dists, uint32_t* seeds = nullptr,
                     size_t num_seeds_per_query = 0) {
        detail::check(grab_index_search_range(h_, host_queries, num_queries, k, range_radius, start_ts, end_ts,
                                              host_indices, host_dists, seeds, num_seeds_per_query));
    }
    void setBuildParams(uint32_t inter_degree, uint32_t graph_degree) {
        detail::check(grab_index_set_build_params(h_, inter_degree, graph_degree));
    }
    void setQueryParams(uint32_t itopk_size, uint32_t search_width, uint32_t min_iterations, uint32_t max_iterations,
                        uint32_t hash_bitlen) {
        detail::check(grab_index_set_query_params(h_, itopk_size, search_width, min_iterations, max_iterations, hash_bitlen));
    }
    void* get_data() { return const_cast<float*>(grab_index_get_data(h_)); }
    void save(const std::string& filepath) { detail::check(grab_index_save(h_, filepath.c_str())); }
    void load(const std::string& filepath) { detail::check(grab_index_load(h_, filepath.c_str())); }
    size_t size() const { return grab_index_size(h_); }

    // ---- additions of this implementation ----
    // one window per query, seeds drawn per query on the device
    void query_range_batch(const float* host_queries, size_t num_queries, int k, const uint64_t* start_ts,
                           const uint64_t* end_ts, int64_t* host_indices, float* host_dists) {
        detail::check(grab_index_search_range_batch(h_, host_queries, num_queries, k, start_ts, end_ts, host_indices, host_dists));
    }
    // the exact top-k of every query inside its window (a scan of the window's rows, not a graph search); k <= 128
    void scan_range_batch(const float* host_queries, size_t num_queries, int k, const uint64_t* start_ts,
                          const uint64_t* end_ts, int64_t* host_indices, float* host_dists) {
        detail::check(grab_index_scan_range_batch(h_, host_queries, num_queries, k, start_ts, end_ts, host_indices, host_dists));
    }
    // query_range_batch scans windows of at most this fraction of the rows exactly and searches the graph for the others (0 = never)
    void setScanBelow(double fraction) { detail::check(grab_index_set_scan_below(h_, fraction)); }
    // range searches take their seeds from an entry-point layer of num_samples rows (0 = off)
    void setEntryLayer(uint32_t num_samples, uint32_t seeds_per_query = 16) {
        detail::check(grab_index_set_entry_layer(h_, num_samples, seeds_per_query));
    }
    // coarse level of that layer: k-means groups of the sample rows, only the groups of the nearest centroids are scored
    void setEntryGroups(uint32_t num_groups, uint32_t nprobe = 16, uint32_t min_rows = 32) {
        detail::check(grab_index_set_entry_groups(h_, num_groups, nprobe, min_rows));
    }
    // with the coarse level: the in-window rows of the nearest groups go to the search as listed (at most max_rows, 0 = scored)
    void setEntryList(uint32_t max_rows) { detail::check(grab_index_set_entry_list(h_, max_rows)); }
    // query_range_batch cuts batches larger than this into chunks that overlap on the index's streams (0 = never)
    void setBatchChunk(size_t queries_per_chunk) { detail::check(grab_index_set_batch_chunk(h_, queries_per_chunk)); }
    // GRAB_FLAG_* bits applied to every search of this index
    void setFlags(uint32_t flags) { detail::check(grab_index_set_flags(h_, flags)); }
    // replaces the std::random_device draws of the reference by a reproducible generator
    void setSeed(uint64_t seed) { detail::check(grab_index_set_seed(h_, seed)); }
    void setInsertParams(uint32_t itopk_size, uint32_t search_width, uint32_t min_iterations, uint32_t max_iterations,
                         uint32_t hash_bitlen) {
        detail::check(grab_index_set_insert_params(h_, itopk_size, search_width, min_iterations, max_iterations, hash_bitlen));
    }
    const uint32_t* get_graph() { return grab_index_get_graph(h_); }
    grab_index* handle() { return h_; }

private:
    grab_index* h_ = nullptr;
};

}  // namespace cagra
