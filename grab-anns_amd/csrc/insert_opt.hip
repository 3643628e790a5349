// Incremental insert into the time-partitioned graph.  Restates cagra::insert of the partitioned
// index (src/index/cagra_opt.cu:1674-1981) with update_topology_gpu_opt's v1 branch
// (src/index/insert.cu:444-727, :1398-1529): search the old graph twice with the new rows as
// queries (all slots, unseeded; local slots only, seeded inside the bucket), merge the nearest rows
// of the batch itself into the bucket result, write the new rows (local slots from the bucket
// list, remote slots from the global list) and let every old row that was chosen take the new row
// into a pseudo-random slot of the matching part of its own row.
#include <algorithm>

#include "device_sort.hpp"
#include "insert_internal.hpp"
#include "search_internal.hpp"

namespace grab {
using namespace dev;
namespace {

constexpr uint32_t kMaxBatch = 1024;  // rows of one call; also the longest merged list (merge_topk_kernel, cagra_opt.cu:1529-1591)

// cagra_opt.cu:1847-1915: the tmp_size nearest rows of the batch (ids shifted by n_existing) join
// the bucket search's list and the first search_k of the union stay (merge_topk_kernel, :1475-1527).
// The reference takes the batch distances from a brute-force library call and orders ties by its
// sorting network; here both lists carry the same 8-lane distance and order by (distance, id).
template <int METRIC>
__global__ void __launch_bounds__(256) merge_batch_kernel(const float* __restrict__ new_data, uint32_t n_new, uint32_t dim,
                                                          uint32_t n_existing, uint32_t search_k, uint32_t tmp_size,
                                                          int64_t* __restrict__ local_ids, const float* __restrict__ local_dists) {
    __shared__ uint64_t batch[kMaxBatch];
    __shared__ uint64_t all[kMaxBatch];
    const uint32_t row = blockIdx.x;
    const float* q = new_data + (size_t)row * dim;
    const int grp = threadIdx.x >> 3, j8 = threadIdx.x & 7;
    for (uint32_t j0 = 0; j0 < n_new; j0 += 32) {
        const uint32_t j = j0 + grp;
        if (j < n_new) {  // uniform per group of 8 lanes
            const float d = group8_distance<METRIC>(q, new_data + (size_t)j * dim, dim, j8);
            if (j8 == 0) batch[j] = make_sel_key(d, n_existing + j);
        }
    }
    int64_t* mine = local_ids + (size_t)row * search_k;
    const uint32_t total = search_k + tmp_size;
    for (uint32_t s = threadIdx.x; s < total; s += 256) {
        uint64_t key = kInvalidKey;
        if (s < search_k) {
            const int64_t id = mine[s];
            if (id >= 0 && id < (int64_t)n_existing) key = make_sel_key(local_dists[(size_t)row * search_k + s], (uint32_t)id);
        }
        all[s] = key;
    }
    __syncthreads();
    for (uint32_t j = threadIdx.x; j < n_new; j += 256) {
        const uint64_t key = batch[j];
        uint32_t rank = 0;
        for (uint32_t x = 0; x < n_new; ++x) rank += batch[x] < key;
        if (rank < tmp_size) all[search_k + rank] = key;
    }
    for (uint32_t s = threadIdx.x; s < search_k; s += 256) mine[s] = -1;
    __syncthreads();
    for (uint32_t s = threadIdx.x; s < total; s += 256) {
        const uint64_t key = all[s];
        if (key == kInvalidKey) continue;
        // the strict traversal can leave an id twice in the bucket's list: equal keys keep both places, by position
        uint32_t rank = 0;
        for (uint32_t x = 0; x < total; ++x) rank += (all[x] < key || (all[x] == key && x < s)) ? 1u : 0u;
        if (rank < search_k) mine[rank] = (int64_t)(uint32_t)(key & 0xFFFFFFFFull);
    }
}

// fill_new_nodes_kernel_opt, insert.cu:444-566, one wave per new row (one thread there).  The lists are walked 64
// candidates at a time: the tests of a chunk (and the timestamp reads behind them) run in parallel, a ballot gives
// every accepted candidate the slot that the sequential walk would have given it, and the walk stops as soon as the
// slots are full.  The second local pass of the reference (:510-522) differs from the first only for ids of 2^31 and
// above, which no index here can hold, and finds nothing the first left: it is not repeated.  The row starts as
// 0xFFFFFFFF (the reference leaves what the fresh mapping holds); ids outside the graph are passed over (the
// reference reads their timestamp out of bounds).
__global__ void __launch_bounds__(64) fill_new_rows_kernel(uint32_t* __restrict__ graph, const uint64_t* __restrict__ ts,
                                                           int64_t* __restrict__ local_ids, int64_t* __restrict__ global_ids,
                                                           uint32_t n_existing, uint32_t n_new, uint32_t total_degree,
                                                           uint32_t local_degree, uint32_t search_k) {
    __shared__ uint32_t loc[GRAB_MAX_DEGREE];  // the local slots as filled
    const uint32_t t = blockIdx.x;
    const int lane = threadIdx.x;
    const uint64_t lt = (1ull << lane) - 1ull;
    const uint32_t me = n_existing + t;
    const int64_t n_total = (int64_t)n_existing + n_new;
    const uint64_t my_ts = ts[me];
    uint32_t* row = graph + (size_t)me * total_degree;
    int64_t* lc = local_ids + (size_t)t * search_k;
    int64_t* gc = global_ids + (size_t)t * search_k;
    for (uint32_t x = lane; x < total_degree; x += 64) row[x] = kInvalidId;
    uint32_t filled = 0;  // wave-uniform
    for (uint32_t k0 = 0; k0 < search_k && filled < local_degree; k0 += 64) {  // :471-507
        const uint32_t k = k0 + lane;
        const int64_t c = k < search_k ? lc[k] : -1;
        const bool ok = c >= 0 && c < n_total && (uint32_t)c != me && ts[c] == my_ts;
        const uint64_t b = __ballot(ok);
        const uint32_t slot = filled + (uint32_t)__popcll(b & lt);
        if (ok && slot < local_degree) {
            row[slot] = (uint32_t)c;
            loc[slot] = (uint32_t)c;
            lc[k] = -1;
        }
        filled = min(filled + (uint32_t)__popcll(b), local_degree);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    uint32_t filled_remote = 0;
    const uint32_t max_remote = total_degree - local_degree;
    for (uint32_t k0 = 0; k0 < search_k && filled_remote < max_remote; k0 += 64) {  // :528-553
        const uint32_t k = k0 + lane;
        const int64_t c = k < search_k ? gc[k] : -1;
        bool ok = c >= 0 && c < n_total && (uint32_t)c != me;
        if (ok) {
            bool in_local = false;
            for (uint32_t x = 0; x < filled; ++x) in_local |= loc[x] == (uint32_t)c;
            ok = !in_local && ts[c] != my_ts;
        }
        const uint64_t b = __ballot(ok);
        const uint32_t slot = filled_remote + (uint32_t)__popcll(b & lt);
        if (ok && slot < max_remote) {
            row[local_degree + slot] = (uint32_t)c;
            gc[k] = -1;
        }
        filled_remote = min(filled_remote + (uint32_t)__popcll(b), max_remote);
    }
    for (uint32_t k0 = 0; k0 < search_k && filled_remote < max_remote; k0 += 64) {  // :556-565
        const uint32_t k = k0 + lane;
        const int64_t c = k < search_k ? gc[k] : -1;  // this lane's own marks of the walk above are in place
        const bool ok = c >= 0 && c < n_total && (uint32_t)c != me;
        const uint64_t b = __ballot(ok);
        const uint32_t slot = filled_remote + (uint32_t)__popcll(b & lt);
        if (ok && slot < max_remote) {
            row[local_degree + slot] = (uint32_t)c;
            gc[k] = -1;
        }
        filled_remote = min(filled_remote + (uint32_t)__popcll(b), max_remote);
    }
}

// generate_update_requests_kernel_opt, insert.cu:568-635.  A request is the key
// (target*2 + kind) << 32 | (new row, slot): sorted, the requests of one target are together, the
// local ones (kind 0) before the remote ones (kind 1), each kind by ascending (new row, slot) - the
// reference's mailboxes hold them in atomic arrival order.  Targets among the new rows are left
// out: the reference counts them and never applies them (:654).
__global__ void __launch_bounds__(256) requests_kernel(const uint32_t* __restrict__ graph, const uint64_t* __restrict__ ts,
                                                       uint32_t n_existing, uint32_t n_new, uint64_t target_ts,
                                                       uint32_t total_degree, uint32_t local_degree,
                                                       uint64_t* __restrict__ requests, uint32_t padded) {
    const uint32_t t = blockIdx.x * 256 + threadIdx.x;
    if (t >= padded) return;
    uint64_t key = kInvalidKey;
    if (t < n_new * total_degree) {
        const uint32_t slot = t % total_degree;
        const uint32_t dest = graph[(size_t)n_existing * total_degree + t];
        if (dest < n_existing) {
            const uint32_t kind = slot < local_degree ? 0u : 1u;
            if (kind == 0 || ts[dest] != target_ts) key = ((uint64_t)(dest * 2u + kind) << 32) | t;  // :626-628
        }
    }
    requests[t] = key;
}

// insert.cu:637-644
__device__ __forceinline__ uint32_t wang_hash(uint32_t seed) {
    seed = (seed ^ 61u) ^ (seed >> 16);
    seed *= 9u;
    seed = seed ^ (seed >> 4);
    seed *= 0x27d4eb2du;
    seed = seed ^ (seed >> 15);
    return seed;
}

// apply_topology_updates_kernel_opt, insert.cu:646-727: the first request of a target walks the
// target's requests.  Local ones (at most local_degree/2) land in a random slot of the local part,
// one time in ten in its first half; remote ones (at most (total-local)/2) land in the first third
// of the remote part when the timestamps are at most 20 apart, else in the rest.
__global__ void __launch_bounds__(256) apply_requests_kernel(uint32_t* __restrict__ graph, const uint64_t* __restrict__ ts,
                                                             const uint64_t* __restrict__ sorted, uint32_t total,
                                                             uint32_t n_existing, uint32_t total_degree, uint32_t local_degree) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const uint64_t key = sorted[i];
    if (key == kInvalidKey) return;
    const uint32_t target = (uint32_t)(key >> 33);
    if (i != 0 && (uint32_t)(sorted[i - 1] >> 33) == target) return;  // not the leader
    uint32_t* row = graph + (size_t)target * total_degree;
    const uint32_t local_max = local_degree / 2, remote_degree = total_degree - local_degree;
    const uint32_t remote_max = remote_degree / 2;  // insert.cu:1470-1471
    const uint32_t local_half = local_degree / 2, near_len = remote_degree / 3;
    const int64_t my_ts = (int64_t)ts[target];
    uint32_t rng = wang_hash(target);
    uint32_t taken_local = 0, taken_remote = 0;
    for (uint32_t idx = i; idx < total; ++idx) {
        const uint64_t kx = sorted[idx];
        if (kx == kInvalidKey || (uint32_t)(kx >> 33) != target) break;
        const uint32_t kind = (uint32_t)(kx >> 32) & 1u;
        if ((kind ? taken_remote++ : taken_local++) >= (kind ? remote_max : local_max)) continue;  // the mailbox was full
        const uint32_t cand = n_existing + (uint32_t)(kx & 0xFFFFFFFFull) / total_degree;
        uint32_t start, len;
        if (kind == 0) {
            rng = wang_hash(rng);
            const bool strong = (rng % 100u) < 10u;
            start = strong ? 0 : local_half;
            len = strong ? local_half : local_degree - local_half;
        } else {
            const int64_t theirs = (int64_t)ts[cand];
            const bool nearby = theirs >= my_ts - 20 && theirs <= my_ts + 20;  // :706
            start = nearby ? local_degree : local_degree + near_len;
            len = nearby ? near_len : remote_degree - near_len;
        }
        if (len > 0) {
            rng = wang_hash(rng);
            row[start + rng % len] = cand;
        }
    }
}

}  // namespace

size_t insert_partitioned_workspace_bytes(size_t num_new, uint32_t search_k, uint32_t total_degree) {
    const size_t res = num_new * search_k;
    const size_t padded = grab_next_power_of_2((uint32_t)std::max<size_t>(num_new * total_degree, 2));
    return 2 * res * sizeof(int64_t) + 2 * res * sizeof(float) + 2 * padded * sizeof(uint64_t) + 256;
}

int insert_partitioned_impl(const float* d_dataset, uint32_t* d_graph, const uint64_t* d_ts, const uint32_t* d_seeds,
                            size_t num_existing, size_t num_new, uint64_t target_ts, uint32_t dim, uint32_t total_degree,
                            uint32_t local_degree, grab_search_params params, uint32_t num_seeds_per_query, int metric,
                            uint64_t* rng_state, uint32_t flags, void* workspace, hipStream_t st, const SideStream* side) {
    if (num_new == 0) return GRAB_OK;
    GRAB_REQUIRE(d_dataset && d_graph && d_ts && rng_state && workspace, "null pointer");
    GRAB_REQUIRE(num_existing > 0, "insert needs an existing graph");
    GRAB_REQUIRE(total_degree >= 2 && total_degree <= GRAB_MAX_DEGREE, "total_degree %u out of range", total_degree);
    GRAB_REQUIRE(local_degree >= 1 && local_degree < total_degree, "local_degree must be in [1, total_degree)");
    GRAB_REQUIRE(num_seeds_per_query == 0 || d_seeds, "seeds missing");
    GRAB_REQUIRE(num_new <= kMaxBatch, "at most %u rows per call", kMaxBatch);
    const uint32_t search_k = params.itopk_size;  // cagra_opt.cu:1693
    GRAB_REQUIRE(search_k >= 1, "itopk_size must be positive");
    const uint32_t n_existing = (uint32_t)num_existing, n_new = (uint32_t)num_new;
    const uint32_t tmp_size = std::min(n_new, search_k / 2);  // cagra_opt.cu:1853
    GRAB_REQUIRE(search_k + tmp_size <= kMaxBatch, "itopk_size %u too large for the merged list", search_k);
    GRAB_REQUIRE(num_existing + num_new < (1ull << 31), "index too large");

    const size_t res = (size_t)n_new * search_k;
    const uint32_t total = n_new * total_degree;
    const uint32_t padded = grab_next_power_of_2(std::max(total, 2u));
    char* ws = static_cast<char*>(workspace);
    int64_t* gi = reinterpret_cast<int64_t*>(ws);
    int64_t* li = gi + res;
    uint64_t* requests = reinterpret_cast<uint64_t*>(li + res);
    uint64_t* sorted = requests + padded;
    float* gd = reinterpret_cast<float*>(sorted + padded);
    float* ld = gd + res;
    const float* d_queries = d_dataset + num_existing * dim;

    const uint64_t mask_global = splitmix64(rng_state) & 0xFFFFFFFFull;
    const uint64_t mask_local = splitmix64(rng_state) & 0xFFFFFFFFull;
    grab_search_desc d;
    fill_search_desc(&d, GRAB_WRAP_SEARCH_OPT, d_dataset, num_existing, dim, d_graph, total_degree, total_degree, d_queries,
                     num_new, search_k, params, metric, nullptr, 0, mask_global, flags, gi, gd, st);  // :1712-1727
    hipStream_t st_bucket = st;
    if (side != nullptr) {  // everything queued on `st` so far (the graph as the step before left it) comes first
        GRAB_HIP(hipEventRecord(side->fork, st));
        GRAB_HIP(hipStreamWaitEvent(side->stream, side->fork, 0));
        st_bucket = side->stream;
    }
    GRAB_TRY(search_ex_impl(&d, false));
    fill_search_desc(&d, GRAB_WRAP_BUCKET, d_dataset, num_existing, dim, d_graph, total_degree, local_degree, d_queries,
                     num_new, search_k, params, metric, d_seeds, num_seeds_per_query, mask_local, flags, li, ld, st_bucket);  // :1764-1780
    GRAB_TRY(search_ex_impl(&d, false));
    if (side != nullptr) {
        GRAB_HIP(hipEventRecord(side->join, side->stream));
        GRAB_HIP(hipStreamWaitEvent(st, side->join, 0));
    }

    if (metric == kMetricIP)
        hipLaunchKernelGGL(merge_batch_kernel<kMetricIP>, dim3(n_new), dim3(256), 0, st, d_queries, n_new, dim, n_existing,
                           search_k, tmp_size, li, ld);
    else
        hipLaunchKernelGGL(merge_batch_kernel<kMetricL2>, dim3(n_new), dim3(256), 0, st, d_queries, n_new, dim, n_existing,
                           search_k, tmp_size, li, ld);
    hipLaunchKernelGGL(fill_new_rows_kernel, dim3(n_new), dim3(64), 0, st, d_graph, d_ts, li, gi, n_existing, n_new,
                       total_degree, local_degree, search_k);
    hipLaunchKernelGGL(requests_kernel, dim3((padded + 255) / 256), dim3(256), 0, st, d_graph, d_ts, n_existing, n_new,
                       target_ts, total_degree, local_degree, requests, padded);
    GRAB_HIP(hipGetLastError());
    GRAB_TRY(rank_sort_u64_async(requests, sorted, padded, st));
    hipLaunchKernelGGL(apply_requests_kernel, dim3((total + 255) / 256), dim3(256), 0, st, d_graph, d_ts, sorted, total,
                       n_existing, total_degree, local_degree);
    GRAB_HIP(hipGetLastError());
    return GRAB_OK;
}

}  // namespace grab

using namespace grab;

extern "C" int grab_insert_partitioned(const float* d_dataset, uint32_t* d_graph, const uint64_t* d_ts, const uint32_t* d_seeds,
                                       size_t num_existing, size_t num_new, uint64_t target_ts, uint32_t dim,
                                       uint32_t total_degree, uint32_t local_degree, grab_search_params params,
                                       uint32_t num_seeds_per_query, int metric, uint64_t* rng_state, uint32_t flags,
                                       void* stream) {
    if (num_new == 0) return GRAB_OK;
    GRAB_REQUIRE(params.itopk_size >= 1 && params.itopk_size <= kMaxBatch, "itopk_size out of range");
    GRAB_REQUIRE(total_degree >= 2 && total_degree <= GRAB_MAX_DEGREE, "total_degree %u out of range", total_degree);
    GRAB_REQUIRE(num_new <= kMaxBatch, "at most %u rows per call", kMaxBatch);
    DeviceScratch ws;
    GRAB_HIP(ws.alloc(insert_partitioned_workspace_bytes(num_new, params.itopk_size, total_degree)));
    hipStream_t st = static_cast<hipStream_t>(stream);
    GRAB_TRY(insert_partitioned_impl(d_dataset, d_graph, d_ts, d_seeds, num_existing, num_new, target_ts, dim, total_degree,
                                     local_degree, params, num_seeds_per_query, metric, rng_state, flags, ws.ptr, st));
    GRAB_HIP(hipStreamSynchronize(st));
    return GRAB_OK;
}
