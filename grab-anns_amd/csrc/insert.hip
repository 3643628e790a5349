// Incremental insert into the global graph.  Restates cagra::insert
// (src/index/cagra.cu:938-1015) with find_near_nodes and update_topology_gpu_v1
// (src/index/insert.cu:140-440): search the old graph with the new rows as queries, re-score
// and sort the results, write the new rows, then let every old node that was found take the
// new node into a pseudo-random slot of its own row.
#include <algorithm>

#include "device_sort.hpp"
#include "insert_internal.hpp"
#include "search_internal.hpp"

namespace grab {
using namespace dev;
namespace {

// insert_refine_kernel_warp + insert_sort_kernel (insert.cu:24-72, :80-133), one workgroup per new
// row: its four waves score the result list 32 entries at a time (8 lanes per entry), the first wave
// sorts.  Ids outside [0, n_existing) score kDistMax; the sort carries ids as uint32 and widens
// them again (insert.cu:106,129).  With `striped` the output slot p = lane32 + e*32 receives
// the element of sorted rank lane32*per_lane + e, which is what the reference's striped load
// into a blocked 32-lane network produces (insert.cu:104 against bitonic.cuh:74).
template <int METRIC, int NPL>
__global__ void __launch_bounds__(256) insert_refine_sort_kernel(const float* __restrict__ data, const float* __restrict__ new_data,
                                                                 uint32_t dim, uint32_t n_existing, uint32_t n_new,
                                                                 uint32_t search_k, int64_t* __restrict__ ids, int striped,
                                                                 uint32_t per_lane32) {
    __shared__ uint64_t mykeys[64 * NPL];
    const int lane = threadIdx.x & 63;
    const uint32_t row = blockIdx.x;
    int64_t* myids = ids + (size_t)row * search_k;
    const float* q = new_data + (size_t)row * dim;
    const int grp = threadIdx.x >> 3, j = threadIdx.x & 7;
    for (uint32_t g = threadIdx.x; g < 64u * NPL; g += 256) mykeys[g] = kInvalidKey;
    __syncthreads();
    for (uint32_t c0 = 0; c0 < search_k; c0 += 32) {
        const uint32_t c = c0 + grp;
        if (c < search_k) {  // uniform per group of 8 lanes
            const int64_t id = myids[c];
            float d = kDistMax;
            if (id >= 0 && id < (int64_t)n_existing) d = group8_distance<METRIC>(q, data + (size_t)id * dim, dim, j);
            if (j == 0) mykeys[c] = make_sel_key(d, (uint32_t)id);
        }
    }
    __syncthreads();
    if (threadIdx.x >= 64) return;
    uint64_t k[NPL];
#pragma unroll
    for (int i = 0; i < NPL; ++i) k[i] = mykeys[lane * NPL + i];
    wave_bitonic_sort<NPL>(k);
#pragma unroll
    for (int i = 0; i < NPL; ++i) mykeys[lane * NPL + i] = k[i];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    for (uint32_t p = lane; p < search_k; p += 64) {
        uint32_t src = p;
        if (striped) src = (p & 31u) * per_lane32 + (p >> 5);
        // ranks past search_k are the (FLT_MAX, 0xFFFFFFFF) padding of the reference's network
        const uint64_t kk = src < search_k ? mykeys[src] : kInvalidKey;
        myids[p] = (int64_t)(uint32_t)(kk & 0xFFFFFFFFull);
    }
}

// fill_new_nodes_kernel (insert.cu:225-257) and generate_update_requests_kernel (:263-290)
// in one pass over the sorted results.  A request is the 64-bit key target<<32 | request
// index: sorting the keys groups requests by target and keeps their original order inside a
// group, which is what a stable sort_by_key on the 32-bit target gives (:422-424).
__global__ void __launch_bounds__(256) fill_and_request_kernel(uint32_t* __restrict__ graph, const int64_t* __restrict__ ids,
                                                               uint32_t n_existing, uint32_t n_new, uint32_t degree,
                                                               uint32_t search_k, uint64_t* __restrict__ requests,
                                                               uint32_t padded) {
    const uint32_t t = blockIdx.x * 256 + threadIdx.x;
    const uint32_t total = n_new * search_k;
    if (t >= padded) return;
    if (t >= total) {
        requests[t] = kInvalidKey;
        return;
    }
    const uint32_t i = t / search_k, kk = t - i * search_k;
    const int64_t id = ids[t];
    const bool old_node = id >= 0 && id < (int64_t)n_existing;
    if (kk < degree) graph[(size_t)(n_existing + i) * degree + kk] = old_node ? (uint32_t)id : kInvalidId;
    requests[t] = old_node ? (((uint64_t)(uint32_t)id << 32) | t) : kInvalidKey;
}

// new rows wider than the result list keep 0xFFFFFFFF in the slots past search_k (insert.cu:245)
__global__ void __launch_bounds__(256) fill_tail_kernel(uint32_t* __restrict__ graph, uint32_t n_existing, uint32_t n_new,
                                                        uint32_t degree, uint32_t search_k) {
    const uint32_t t = blockIdx.x * 256 + threadIdx.x;
    const uint32_t width = degree - search_k;
    if (t >= n_new * width) return;
    const uint32_t i = t / width, kk = search_k + (t - i * width);
    graph[(size_t)(n_existing + i) * degree + kk] = kInvalidId;
}

// apply_topology_updates_kernel (insert.cu:296-368): the first request of each target walks
// the target's requests in order; a new id that is not yet in the row overwrites a slot
// drawn from a 64-bit LCG seeded with target*0x9e3779b97f4a7c15 + position of the leader:
// one time in ten a slot of the first half, otherwise one of the second half.
__global__ void __launch_bounds__(256) apply_updates_kernel(uint32_t* __restrict__ graph, const uint64_t* __restrict__ sorted,
                                                            uint32_t total, uint32_t degree, uint32_t n_existing,
                                                            uint32_t search_k) {
    const uint32_t tid = blockIdx.x * 256 + threadIdx.x;
    if (tid >= total) return;
    const uint64_t key = sorted[tid];
    if (key == kInvalidKey) return;
    const uint32_t target = (uint32_t)(key >> 32);
    if (tid != 0 && (uint32_t)(sorted[tid - 1] >> 32) == target) return;  // not the leader
    uint32_t* nb = graph + (size_t)target * degree;
    const uint32_t num_protected = degree / 2, num_unprotected = degree - num_protected;
    uint64_t rng = (uint64_t)target * 0x9e3779b97f4a7c15ull + (uint64_t)tid;
    for (uint32_t idx = tid; idx < total; ++idx) {
        const uint64_t kx = sorted[idx];
        if (kx == kInvalidKey || (uint32_t)(kx >> 32) != target) break;
        const uint32_t nid = n_existing + (uint32_t)(kx & 0xFFFFFFFFull) / search_k;
        // the whole row is requested at once (no early exit): one memory latency per request, not one per slot
        bool exists = false;
        if ((degree & 3u) == 0) {
            const uint4* nb4 = reinterpret_cast<const uint4*>(nb);
#pragma unroll 16
            for (uint32_t x = 0; x < degree / 4; ++x) {
                const uint4 v = nb4[x];
                exists |= (v.x == nid) | (v.y == nid) | (v.z == nid) | (v.w == nid);
            }
        } else {
            for (uint32_t x = 0; x < degree; ++x) exists |= nb[x] == nid;
        }
        if (exists) continue;
        rng = rng * 6364136223846793005ull + 1;
        const uint32_t r1 = (uint32_t)(rng >> 32);
        const bool upd_protected = (r1 % 10u == 0);
        rng = rng * 6364136223846793005ull + 1;
        const uint32_t r2 = (uint32_t)(rng >> 32);
        const uint32_t slot = upd_protected ? (r2 % num_protected) : num_protected + (r2 % num_unprotected);
        nb[slot] = nid;
    }
}

template <int METRIC>
int launch_refine_sort(const float* data, const float* new_data, uint32_t dim, uint32_t n_existing, uint32_t n_new,
                       uint32_t search_k, int64_t* ids, int striped, hipStream_t st) {
    const uint32_t grid = n_new;
    const uint32_t per_lane32 = search_k <= 64 ? 2 : search_k <= 128 ? 4 : search_k <= 256 ? 8 : 16;  // insert.cu:204-213
#define GRAB_RS(NPL) \
    hipLaunchKernelGGL((insert_refine_sort_kernel<METRIC, NPL>), dim3(grid), dim3(256), 0, st, data, new_data, dim, n_existing, n_new, search_k, ids, striped, per_lane32)
    if (search_k <= 64) GRAB_RS(1);
    else if (search_k <= 128) GRAB_RS(2);
    else if (search_k <= 256) GRAB_RS(4);
    else if (search_k <= 512) GRAB_RS(8);
    else GRAB_RS(16);
#undef GRAB_RS
    GRAB_HIP(hipGetLastError());
    return GRAB_OK;
}

}  // namespace

size_t insert_workspace_bytes(size_t num_new, uint32_t degree) {
    const size_t search_k = (size_t)degree * 2;
    const size_t total = num_new * search_k;
    const size_t padded = grab_next_power_of_2((uint32_t)std::max<size_t>(total, 2));
    return total * sizeof(int64_t) + total * sizeof(float) + 2 * padded * sizeof(uint64_t) + 256;
}

int insert_impl(const float* d_dataset, uint32_t dim, size_t num_existing, size_t num_new, const float* d_new_data,
                uint32_t* d_graph, uint32_t degree, grab_search_params params, int metric, uint64_t* rng_state,
                uint32_t flags, int striped_sort, void* workspace, hipStream_t st) {
    if (num_new == 0) return GRAB_OK;
    GRAB_REQUIRE(d_dataset && d_new_data && d_graph && rng_state && workspace, "null pointer");
    GRAB_REQUIRE(num_existing > 0, "insert needs an existing graph");
    GRAB_REQUIRE(degree >= 1 && degree <= GRAB_MAX_DEGREE, "graph_degree %u out of range", degree);
    const uint32_t search_k = degree * 2;  // cagra.cu:951
    GRAB_REQUIRE(search_k <= 1024, "graph_degree above 512 is not supported");
    GRAB_REQUIRE(num_new * (size_t)search_k < (1ull << 31), "too many new rows in one call");
    GRAB_REQUIRE(num_existing + num_new < (1ull << 31), "index too large");
    const uint32_t n_existing = (uint32_t)num_existing, n_new = (uint32_t)num_new;
    const uint32_t total = n_new * search_k;
    const uint32_t padded = grab_next_power_of_2(std::max(total, 2u));

    char* ws = static_cast<char*>(workspace);
    int64_t* ids = reinterpret_cast<int64_t*>(ws);
    ws += (size_t)total * sizeof(int64_t);
    uint64_t* requests = reinterpret_cast<uint64_t*>(ws);
    ws += (size_t)padded * sizeof(uint64_t);
    uint64_t* sorted = reinterpret_cast<uint64_t*>(ws);
    ws += (size_t)padded * sizeof(uint64_t);
    float* dists = reinterpret_cast<float*>(ws);

    // find_near_nodes (insert.cu:140-219): one search per 64 new rows, each with its own mask
    for (size_t off = 0; off < num_new; off += 64) {
        const size_t cur = std::min<size_t>(64, num_new - off);
        const uint64_t mask = splitmix64(rng_state) & 0xFFFFFFFFull;
        grab_search_desc d;
        fill_search_desc(&d, GRAB_WRAP_SEARCH, d_dataset, num_existing, dim, d_graph, degree, degree,
                         d_new_data + off * dim, cur, search_k, params, metric, nullptr, 0, mask, flags,
                         ids + off * search_k, dists + off * search_k, st);
        GRAB_TRY(search_ex_impl(&d, false));
    }
    if (metric == kMetricIP)
        GRAB_TRY(launch_refine_sort<kMetricIP>(d_dataset, d_new_data, dim, n_existing, n_new, search_k, ids, striped_sort, st));
    else
        GRAB_TRY(launch_refine_sort<kMetricL2>(d_dataset, d_new_data, dim, n_existing, n_new, search_k, ids, striped_sort, st));

    hipLaunchKernelGGL(fill_and_request_kernel, dim3((padded + 255) / 256), dim3(256), 0, st, d_graph, ids, n_existing, n_new,
                       degree, search_k, requests, padded);
    if (degree > search_k)
        hipLaunchKernelGGL(fill_tail_kernel, dim3((n_new * (degree - search_k) + 255) / 256), dim3(256), 0, st, d_graph,
                           n_existing, n_new, degree, search_k);
    GRAB_TRY(rank_sort_u64_async(requests, sorted, padded, st));
    hipLaunchKernelGGL(apply_updates_kernel, dim3((total + 255) / 256), dim3(256), 0, st, d_graph, sorted, total, degree,
                       n_existing, search_k);
    GRAB_HIP(hipGetLastError());
    return GRAB_OK;
}

}  // namespace grab

using namespace grab;

extern "C" {

int grab_insert(const float* d_dataset, uint32_t dim, size_t num_existing, size_t num_new, const float* d_new_data,
                uint32_t* d_graph, uint32_t graph_degree, grab_search_params params, int metric, uint64_t* rng_state,
                uint32_t flags, int striped_sort, void* stream) {
    if (num_new == 0) return GRAB_OK;
    GRAB_REQUIRE(graph_degree >= 1 && graph_degree <= GRAB_MAX_DEGREE, "graph_degree %u out of range", graph_degree);
    DeviceScratch ws;
    GRAB_HIP(ws.alloc(insert_workspace_bytes(num_new, graph_degree)));
    hipStream_t st = static_cast<hipStream_t>(stream);
    GRAB_TRY(insert_impl(d_dataset, dim, num_existing, num_new, d_new_data, d_graph, graph_degree, params, metric, rng_state,
                         flags, striped_sort, ws.ptr, st));
    GRAB_HIP(hipStreamSynchronize(st));
    return GRAB_OK;
}

}  // extern "C"
