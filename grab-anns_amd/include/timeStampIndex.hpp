// timestamp::TimeStampIndex with the reference's public surface (src/timeStampIndex.cuh:47-63) as a
// header-only shell over the C ABI: one CagraIndex per timestamp, a virtual index over k-means centroids
// of the buckets, vote-and-probe queries.  query_by_timestamp is declared by the reference
// (src/timeStampIndex.cuh:59-61) but never defined there; it is not offered here either.
#pragma once
#include <cstdint>
#include <stdexcept>

#include "cagra.hpp"
#include "grab_anns.h"

namespace timestamp {

class TimeStampIndex {
public:
    TimeStampIndex(uint32_t dim, uint32_t degree = 32, size_t cluster_ratio = 1000) {
        cagra::detail::check(grab_tsindex_create(dim, degree, cluster_ratio, 0, &h_));
    }
    ~TimeStampIndex() { grab_tsindex_destroy(h_); }
    TimeStampIndex(const TimeStampIndex&) = delete;
    TimeStampIndex& operator=(const TimeStampIndex&) = delete;

    // returns the global id of the first inserted vector; ids are consecutive in arrival order
    uint64_t insert(const float* vectors, const uint64_t* timestamps, size_t num_vectors) {
        uint64_t start = 0;
        cagra::detail::check(grab_tsindex_insert(h_, vectors, timestamps, num_vectors, &start));
        return start;
    }
    void build_virtual_index() { cagra::detail::check(grab_tsindex_build_virtual_index(h_)); }
    // one query vector; unfilled slots are -1 / -1.0f
    void query(const float* query, size_t topk, int64_t* out_indices, float* out_dists, int probe_buckets = 5) {
        cagra::detail::check(grab_tsindex_query(h_, query, topk, out_indices, out_dists, probe_buckets));
    }
    size_t size() const { return grab_tsindex_size(h_); }
    grab_tsindex* handle() { return h_; }

private:
    grab_tsindex* h_ = nullptr;
};

}  // namespace timestamp
