// Insert path shared between the stateless entry point and the index handle.
#pragma once
#include "common.hpp"
#include "device_utils.hpp"

namespace grab {

// bytes of device workspace that one insert_impl call with `num_new` rows needs
size_t insert_workspace_bytes(size_t num_new, uint32_t degree);

// Enqueues one cagra::insert step on `st` without synchronising.  `workspace` is device
// memory of at least insert_workspace_bytes(num_new, degree).
int insert_impl(const float* d_dataset, uint32_t dim, size_t num_existing, size_t num_new, const float* d_new_data,
                uint32_t* d_graph, uint32_t degree, grab_search_params params, int metric, uint64_t* rng_state,
                uint32_t flags, int striped_sort, void* workspace, hipStream_t st);

// the same for one cagra::insert step of the time-partitioned index (src/index/cagra_opt.cu:1674-1981);
// the new rows and their timestamps are already at [num_existing, num_existing + num_new)
size_t insert_partitioned_workspace_bytes(size_t num_new, uint32_t search_k, uint32_t total_degree);
// A second stream (default priority) and the two events that fork it from and join it to the caller's stream.
struct SideStream {
    hipStream_t stream = nullptr;
    hipEvent_t fork = nullptr, join = nullptr;
};
// `side` (may be null): the bucket search of a step runs there, beside the search of the whole graph - the two are
// independent and a step's 32 queries leave most of the device idle.
int insert_partitioned_impl(const float* d_dataset, uint32_t* d_graph, const uint64_t* d_ts, const uint32_t* d_seeds,
                            size_t num_existing, size_t num_new, uint64_t target_ts, uint32_t dim, uint32_t total_degree,
                            uint32_t local_degree, grab_search_params params, uint32_t num_seeds_per_query, int metric,
                            uint64_t* rng_state, uint32_t flags, void* workspace, hipStream_t st,
                            const SideStream* side = nullptr);

}  // namespace grab
