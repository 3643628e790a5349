// cagra::CagraIndexOpt (src/cagraIndexOpt.cuh:13-155) over the C ABI: add / build / query / query_local /
// query_range with the reference's signatures.  build() makes the time-partitioned graph
// (src/index/cagra_opt.cu:928-1106): timestamps are bucket indices 0..B-1 and rows arrive grouped by
// bucket.  insert() is the mailbox insert of the partitioned graph (src/cagraIndexOpt.cu:557-652, the v1
// topology update of src/index/insert.cu:444-727); insert_global() is the global-graph insert of
// cagra::CagraIndex.  save/load use the reference's "MCAG" file layout.
#pragma once
#include <cstdint>
#include <string>
#include <vector>

#include "cagra.hpp"
#include "grab_anns.h"

namespace cagra {

class CagraIndexOpt {
public:
    CagraIndexOpt(uint32_t dim, uint32_t graph_degree = 32, uint32_t local_degree = 16,
                  size_t vmm_max_bytes = 20ULL * 1024 * 1024 * 1024) {
        detail::check(grab_index_create(dim, graph_degree, local_degree, vmm_max_bytes, &h_));
        // src/cagraIndexOpt.cu:32-37
        detail::check(grab_index_set_build_params(h_, graph_degree > 128 ? graph_degree : 128, graph_degree));
        detail::check(grab_index_set_query_params(h_, 256, 6, 1, 50, 13));
    }
    ~CagraIndexOpt() { grab_index_destroy(h_); }
    CagraIndexOpt(const CagraIndexOpt&) = delete;
    CagraIndexOpt& operator=(const CagraIndexOpt&) = delete;

    void add(size_t num_vectors, const float* add_vectors, const uint64_t* add_timestamps) {  // ts mandatory
        if (add_timestamps == nullptr) throw std::runtime_error("CagraIndexOpt::add needs timestamps");
        detail::check(grab_index_add(h_, num_vectors, add_vectors, add_timestamps));
    }
    // time-partitioned graph: local edges inside a timestamp's rows, remote edges in the last slots
    void build() { detail::check(grab_index_build_partitioned(h_)); }
    // one global CAGRA graph over all rows (what cagra::CagraIndex builds)
    void build_global() { detail::check(grab_index_build(h_)); }
    // all rows of one call belong to the bucket insert_timestamps[0]; the query parameters become
    // 128/4/0/100/14 afterwards (src/cagraIndexOpt.cu:581-587)
    void insert(size_t new_vectors, const float* insert_vectors, const uint64_t* insert_timestamps) {
        detail::check(grab_index_insert_partitioned(h_, new_vectors, insert_vectors, insert_timestamps));
    }
    void insert_global(size_t new_vectors, const float* insert_vectors, const uint64_t* insert_timestamps) {
        detail::check(grab_index_insert(h_, new_vectors, insert_vectors, insert_timestamps));
    }
    // min_ts / max_ts are ignored, as in the reference (src/cagraIndexOpt.cu:226-227)
    void query(const float* host_queries, size_t num_queries, int k, uint64_t /*min_ts*/, uint64_t /*max_ts*/,
               int64_t* host_indices, float* host_dists, const uint32_t* seeds = nullptr, size_t num_seeds_per_query = 0) {
        detail::check(grab_index_search(h_, host_queries, num_queries, k, host_indices, host_dists, seeds, num_seeds_per_query));
    }
    // the local_degree argument is overridden by the member, as in the reference (:310)
    void query_local(const float* host_queries, size_t num_queries, int k, uint64_t target_timestamp,
                     int64_t* host_indices, float* host_dists, uint32_t /*local_degree*/ = 0) {
        detail::check(grab_index_search_bucket(h_, host_queries, num_queries, k, target_timestamp, host_indices, host_dists));
    }
    // [start_bucket, end_bucket); -1 / -1.0f when the range is empty (:479-485)
    void query_range(const float* host_queries, size_t num_queries, int k, uint64_t start_bucket, uint64_t end_bucket,
                     int64_t* host_indices, float* host_dists, uint32_t /*local_degree*/ = 0) {
        detail::check(grab_index_search_range(h_, host_queries, num_queries, k, 0.0f, start_bucket, end_bucket,
                                              host_indices, host_dists, nullptr, 0));
    }
    void setBuildParams(uint32_t inter_degree, uint32_t graph_degree) {
        detail::check(grab_index_set_build_params(h_, inter_degree, graph_degree));
    }
    void setQueryParams(uint32_t itopk_size, uint32_t search_width, uint32_t min_iterations, uint32_t max_iterations,
                        uint32_t hash_bitlen) {
        detail::check(grab_index_set_query_params(h_, itopk_size, search_width, min_iterations, max_iterations, hash_bitlen));
    }
    const float* get_data() const { return grab_index_get_data(h_); }
    uint32_t* get_graph() { return const_cast<uint32_t*>(grab_index_get_graph(h_)); }
    std::vector<uint32_t> get_ids_by_timestamp(uint64_t ts) const {
        std::vector<uint32_t> out(grab_index_ids_by_timestamp(h_, ts, nullptr, 0));
        if (!out.empty()) grab_index_ids_by_timestamp(h_, ts, out.data(), out.size());
        return out;
    }
    // inclusive max_ts, as in the reference (src/cagraIndexOpt.cu:95-131)
    std::vector<uint32_t> sample_seeds_by_time(uint64_t min_ts, uint64_t max_ts, size_t num) const {
        std::vector<uint32_t> out(num);
        out.resize(grab_index_sample_seeds_by_time(h_, min_ts, max_ts, num, out.data(), out.size()));
        return out;
    }
    // "MCAG" version 1 file, the reference's layout (src/cagraIndexOpt.cu:725-896)
    void save(const std::string& filepath) { detail::check(grab_index_save_mcag(h_, filepath.c_str())); }
    void load(const std::string& filepath) { detail::check(grab_index_load_mcag(h_, filepath.c_str())); }
    size_t size() const { return grab_index_size(h_); }
    grab_index* handle() { return h_; }

private:
    grab_index* h_ = nullptr;
};

}  // namespace cagra
