// Time-partitioned graph: every bucket of rows (one timestamp) gets a full-width CAGRA graph of its
// own, then the last slots of every row are overwritten with "remote" edges into other buckets and
// reverse remote edges are injected.  Restates build_time_partitioned_graph,
// build_global_remote_edges and enhance_global_connectivity with their kernels
// (src/index/cagra_opt.cu:928-1106, :796-907, :739-793, :209-303, :457-600).  The reference takes
// the global candidates from FAISS IVF-PQ with exact re-ranking and bounces the per-bucket graphs
// through host memory; here candidates are exact (the MFMA contraction) and nothing leaves the device.
#include <algorithm>
#include <vector>

#include "common.hpp"
#include "device_utils.hpp"
#include "graph_internal.hpp"

namespace grab {
using namespace dev;
namespace {

// ids of a bucket's graph are local to the bucket: shift them by the bucket's first row
__global__ void __launch_bounds__(256) shift_ids_kernel(uint32_t* __restrict__ g, size_t count, uint32_t offset) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < count && g[i] != kInvalidId) g[i] += offset;
}

// update_remote_edges_kernel, cagra_opt.cu:209-303: one thread per row walks its global candidates
// (nearest first) three times - other buckets within +-20 % of the bucket range (at most a third of
// the remote slots), then buckets farther away, then whatever other bucket is left.  A used
// candidate is remembered in a bit set (the reference overwrites it in place).
__global__ void __launch_bounds__(256) remote_edges_kernel(uint32_t* __restrict__ graph, const uint64_t* __restrict__ ts,
                                                           const uint32_t* __restrict__ cand, uint32_t n, uint32_t total_degree,
                                                           uint32_t local_degree, uint32_t gk) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    uint32_t* row = graph + (size_t)i * total_degree;
    const uint32_t* c = cand + (size_t)i * gk;
    const uint64_t my = ts[i];
    const uint64_t total_buckets = ts[n - 1] + 1;
    const uint64_t span = total_buckets / 5 > 1 ? total_buckets / 5 : 1;
    const uint64_t lo = my >= span ? my - span : 0;
    const uint64_t hi = my + span >= total_buckets ? total_buckets - 1 : my + span;
    uint64_t used[4] = {0, 0, 0, 0};  // gk <= 256
    int nearby = 0;
    const int nearby_max = (int)(total_degree - local_degree) / 3;
    for (uint32_t k = 0; k < gk && nearby < nearby_max; ++k) {
        const uint32_t id = c[k];
        if (id == i || id >= n) continue;
        const uint64_t t = ts[id];
        if (t == my || t < lo || t > hi) continue;
        row[local_degree + nearby++] = id;
        used[k >> 6] |= 1ull << (k & 63);
    }
    int far = 0;
    const int far_max = (int)(total_degree - local_degree) - nearby;
    for (uint32_t k = 0; k < gk && far < far_max; ++k) {
        const uint32_t id = c[k];
        if (id == i || id >= n || ((used[k >> 6] >> (k & 63)) & 1ull)) continue;
        const uint64_t t = ts[id];
        if (t == my || (t >= lo && t <= hi)) continue;
        row[local_degree + nearby + far++] = id;
        used[k >> 6] |= 1ull << (k & 63);
    }
    for (uint32_t k = 0; k < gk && far < far_max; ++k) {
        const uint32_t id = c[k];
        if (id == i || id >= n || ((used[k >> 6] >> (k & 63)) & 1ull)) continue;
        if (ts[id] == my) continue;
        row[local_degree + nearby + far++] = id;
    }
}

// cagra_opt.cu:34-41
__device__ __forceinline__ uint32_t wang_hash(uint32_t seed) {
    seed = (seed ^ 61u) ^ (seed >> 16);
    seed *= 9u;
    seed = seed ^ (seed >> 4);
    seed *= 0x27d4eb2du;
    seed = seed ^ (seed >> 15);
    return seed;
}

// kern_inject_global_reverse_edges, cagra_opt.cu:488-600: the sources that point at a row through a
// remote slot go into the weak half of the row's remote slots - an empty slot first, else a slot
// drawn with wang_hash - unless the row already has them.
constexpr uint32_t kMaxRev = 32;
__global__ void __launch_bounds__(256) inject_reverse_kernel(uint32_t* __restrict__ graph, const uint32_t* __restrict__ rev,
                                                             const uint32_t* __restrict__ counts, uint32_t n,
                                                             uint32_t total_degree, uint32_t local_degree) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const uint32_t num_remote = total_degree - local_degree;
    const uint32_t num_strong = num_remote / 2, num_weak = num_remote - num_strong;
    uint32_t rc = counts[i];
    if (rc == 0) return;
    if (rc > kMaxRev) rc = kMaxRev;
    uint32_t* row = graph + (size_t)i * total_degree;
    uint32_t* cur = row + local_degree;  // the row belongs to this thread alone
    const uint32_t* mine = rev + (size_t)i * kMaxRev;
    uint32_t rng = wang_hash(i);
    for (uint32_t r = 0; r < rc; ++r) {
        const uint32_t c = mine[r];
        bool exists = false;
        for (uint32_t x = 0; x < total_degree; ++x)
            if (row[x] == c) {
                exists = true;
                break;
            }
        if (exists) continue;
        bool injected = false;
        for (uint32_t w = num_strong; w < num_remote; ++w)
            if (cur[w] == kInvalidId) {
                cur[w] = c;
                injected = true;
                break;
            }
        if (!injected && num_weak > 0) {
            rng = wang_hash(rng);
            cur[num_strong + (rng % num_weak)] = c;
        }
    }
}

}  // namespace
}  // namespace grab

using namespace grab;

extern "C" {

uint32_t grab_remote_global_k(uint32_t total_degree, uint32_t local_degree) {
    uint32_t gk = (total_degree - local_degree) * 4;
    gk = std::max(64u, (gk + 32) - (gk % 32));
    return std::min(256u, gk);
}

int grab_update_remote_edges(uint32_t* d_graph, const uint64_t* d_ts, const uint32_t* d_candidates, size_t num_dataset,
                             uint32_t total_degree, uint32_t local_degree, uint32_t global_k, void* stream) {
    GRAB_REQUIRE(d_graph && d_ts && d_candidates, "null pointer");
    GRAB_REQUIRE(num_dataset > 0 && num_dataset < (1ull << 31), "num_dataset must be in [1, 2^31)");
    GRAB_REQUIRE(local_degree <= total_degree && total_degree <= GRAB_MAX_DEGREE, "bad degrees");
    GRAB_REQUIRE(global_k >= 1 && global_k <= 256, "global_k must be in [1,256]");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint32_t n = (uint32_t)num_dataset;
    hipLaunchKernelGGL(remote_edges_kernel, dim3((n + 255) / 256), dim3(256), 0, st, d_graph, d_ts, d_candidates, n, total_degree,
                       local_degree, global_k);
    GRAB_HIP(hipGetLastError());
    GRAB_HIP(hipStreamSynchronize(st));
    return GRAB_OK;
}

int grab_enhance_global_connectivity(size_t num_dataset, uint32_t* d_graph, uint32_t total_degree, uint32_t local_degree,
                                     void* stream) {
    GRAB_REQUIRE(d_graph != nullptr, "null pointer");
    GRAB_REQUIRE(num_dataset > 0 && num_dataset < (1ull << 31), "num_dataset must be in [1, 2^31)");
    GRAB_REQUIRE(local_degree <= total_degree && total_degree <= GRAB_MAX_DEGREE, "bad degrees");
    if (total_degree == local_degree) return GRAB_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint32_t n = (uint32_t)num_dataset;
    DeviceScratch rev, cnt;
    GRAB_HIP(rev.alloc((size_t)n * kMaxRev * 4));
    GRAB_HIP(cnt.alloc((size_t)n * 4));
    // sources of every row through remote slots, ascending source id (the reference: atomic arrival order)
    GRAB_TRY(reverse_lists(d_graph, n, total_degree, local_degree, total_degree - local_degree, 1, kMaxRev, rev.as<uint32_t>(),
                           cnt.as<uint32_t>(), st));
    hipLaunchKernelGGL(inject_reverse_kernel, dim3((n + 255) / 256), dim3(256), 0, st, d_graph, rev.as<uint32_t>(), cnt.as<uint32_t>(),
                       n, total_degree, local_degree);
    GRAB_HIP(hipGetLastError());
    GRAB_HIP(hipStreamSynchronize(st));
    return GRAB_OK;
}

int grab_build_global_remote_edges(const float* d_dataset, size_t num_dataset, uint32_t dim, uint32_t* d_graph,
                                   const uint64_t* d_ts, uint32_t total_degree, uint32_t local_degree, int metric,
                                   void* stream) {
    GRAB_REQUIRE(d_dataset && d_graph && d_ts, "null pointer");
    GRAB_REQUIRE(local_degree <= total_degree, "local_degree exceeds the graph degree");
    if (total_degree == local_degree) return GRAB_OK;
    const uint32_t gk = grab_remote_global_k(total_degree, local_degree);
    DeviceScratch cand;
    GRAB_HIP(cand.alloc(num_dataset * (size_t)gk * 4));
    GRAB_TRY(grab_generate_knn_graph(d_dataset, num_dataset, dim, gk, metric, cand.as<uint32_t>(), nullptr, stream));
    GRAB_TRY(grab_update_remote_edges(d_graph, d_ts, cand.as<uint32_t>(), num_dataset, total_degree, local_degree, gk, stream));
    return grab_enhance_global_connectivity(num_dataset, d_graph, total_degree, local_degree, stream);
}

int grab_build_time_partitioned_graph(const float* d_dataset, size_t total_num, uint32_t dim, uint32_t* d_graph,
                                      const uint64_t* d_ts, const size_t* bucket_sizes, size_t num_buckets,
                                      uint32_t total_degree, uint32_t local_degree, int metric, void* stream) {
    GRAB_REQUIRE(d_dataset && d_graph && d_ts && bucket_sizes, "null pointer");
    GRAB_REQUIRE(total_num > 0 && total_num < (1ull << 31), "total_num must be in [1, 2^31)");
    GRAB_REQUIRE(local_degree <= total_degree && total_degree >= 1 && total_degree <= GRAB_MAX_DEGREE / 2, "bad degrees");
    size_t sum = 0;
    for (size_t b = 0; b < num_buckets; ++b) sum += bucket_sizes[b];
    GRAB_REQUIRE(sum == total_num, "bucket sizes do not add up to the number of rows");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint32_t inter = total_degree * 2;  // cagra_opt.cu:945
    size_t max_bucket = 0;
    for (size_t b = 0; b < num_buckets; ++b) max_bucket = std::max(max_bucket, bucket_sizes[b]);
    DeviceScratch knn;
    GRAB_HIP(knn.alloc(std::max<size_t>(max_bucket, 1) * inter * 4));
    const grab_build_params bp{inter, total_degree};
    size_t off = 0;
    for (size_t b = 0; b < num_buckets; ++b) {
        const size_t bs = bucket_sizes[b];
        if (bs == 0) continue;
        uint32_t* g = d_graph + off * total_degree;
        GRAB_TRY(grab_generate_knn_graph(d_dataset + off * dim, bs, dim, inter, metric, knn.as<uint32_t>(), nullptr, stream));
        GRAB_TRY(grab_build_graph(d_dataset + off * dim, bs, knn.as<uint32_t>(), bp, g, stream));
        if (off > 0) {
            const size_t count = bs * total_degree;
            hipLaunchKernelGGL(shift_ids_kernel, dim3((uint32_t)((count + 255) / 256)), dim3(256), 0, st, g, count, (uint32_t)off);
            GRAB_HIP(hipGetLastError());
        }
        off += bs;
    }
    GRAB_HIP(hipStreamSynchronize(st));
    return grab_build_global_remote_edges(d_dataset, total_num, dim, d_graph, d_ts, total_degree, local_degree, metric, stream);
}

}  // extern "C"
