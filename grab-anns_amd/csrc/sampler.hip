// Seed sampling for filtered searches with one window per query.
// Takes the place of the host loop of CagraIndex::query_range (src/cagraIndex.cu:270-295),
// which walks the whole timestamp map, draws one std::sample for the batch and copies it to
// every query.  Here each query gets its own seeds, drawn on the device: the ids inside the
// window form a contiguous run of the timestamp-sorted id list (two binary searches); the
// run is cut into n_seeds strata and one id is taken from each.
#include "common.hpp"
#include "device_utils.hpp"

namespace grab {
namespace {

__device__ __forceinline__ uint64_t mix64(uint64_t x) {
    uint64_t z = x + 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

__device__ __forceinline__ uint64_t lower_bound_u64(const uint64_t* a, uint64_t n, uint64_t v) {
    uint64_t lo = 0, hi = n;
    while (lo < hi) {
        const uint64_t mid = (lo + hi) >> 1;
        if (a[mid] < v) lo = mid + 1; else hi = mid;
    }
    return lo;
}

__global__ void __launch_bounds__(256) sample_window_seeds_kernel(const uint64_t* __restrict__ sorted_ts,
                                                                  const uint32_t* __restrict__ ids_by_ts, uint64_t n,
                                                                  const uint64_t* __restrict__ ws_arr,
                                                                  const uint64_t* __restrict__ we_arr, uint64_t ws0,
                                                                  uint64_t we0, int per_query, uint32_t nq,
                                                                  uint32_t n_seeds, uint64_t seed, uint32_t* __restrict__ out) {
    const uint32_t q = blockIdx.x;
    __shared__ uint64_t bounds[2];
    if (threadIdx.x < 2) {
        const uint64_t v = threadIdx.x == 0 ? (per_query ? ws_arr[q] : ws0) : (per_query ? we_arr[q] : we0);
        bounds[threadIdx.x] = lower_bound_u64(sorted_ts, n, v);
    }
    __syncthreads();
    const uint64_t lo = bounds[0], hi = bounds[1] < bounds[0] ? bounds[0] : bounds[1];
    const uint64_t w = hi - lo;
    for (uint32_t i = threadIdx.x; i < n_seeds; i += 256) {
        uint32_t v = dev::kInvalidId;
        if (w <= n_seeds) {
            if (i < w) v = ids_by_ts[lo + i];
        } else {
            const uint64_t b0 = (uint64_t)i * w / n_seeds, b1 = (uint64_t)(i + 1) * w / n_seeds;
            const uint64_t r = mix64(seed ^ ((uint64_t)q * 0x100000001B3ull + i)) % (b1 - b0);
            v = ids_by_ts[lo + b0 + r];
        }
        out[(size_t)q * n_seeds + i] = v;
    }
}

// timestamps that never decrease with the row id: a window [start,end) is the id interval
// [lower_bound(start), lower_bound(end))
__global__ void __launch_bounds__(256) windows_to_id_ranges_kernel(const uint64_t* __restrict__ ts, uint64_t n,
                                                                   const uint64_t* __restrict__ ws, const uint64_t* __restrict__ we,
                                                                   uint32_t nq, uint64_t* __restrict__ lo, uint64_t* __restrict__ hi) {
    __shared__ uint64_t piv[dev::kPivots];
    const uint64_t step = dev::load_pivots(ts, n, piv);
    __syncthreads();
    const uint32_t q = blockIdx.x * 256 + threadIdx.x;
    if (q >= nq) return;
    const uint64_t l = dev::lower_bound_pivots(ts, n, piv, step, ws[q]);
    uint64_t h = dev::lower_bound_pivots(ts, n, piv, step, we[q]);
    if (h < l) h = l;
    lo[q] = l;
    hi[q] = h;
}

__global__ void __launch_bounds__(256) neighbor_timestamps_kernel(const uint32_t* __restrict__ graph, const uint64_t* __restrict__ ts,
                                                                  uint64_t total, uint64_t n, uint64_t* __restrict__ out) {
    const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const uint32_t nb = graph[i];
    out[i] = nb < n ? ts[nb] : ~0ull;
}

__global__ void __launch_bounds__(256) neighbor_ranks_kernel(const uint32_t* __restrict__ graph, const uint32_t* __restrict__ rank,
                                                             uint64_t total, uint64_t n, uint32_t* __restrict__ out) {
    const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const uint32_t nb = graph[i];
    out[i] = nb < n ? rank[nb] : 0xFFFFFFFFu;
}

}  // namespace

int windows_to_id_ranges_async(const uint64_t* d_ts, size_t n, const uint64_t* d_win_start, const uint64_t* d_win_end,
                               size_t nq, uint64_t* d_lo, uint64_t* d_hi, hipStream_t st) {
    GRAB_REQUIRE(d_ts && d_win_start && d_win_end && d_lo && d_hi, "null pointer");
    if (nq == 0) return GRAB_OK;
    hipLaunchKernelGGL(windows_to_id_ranges_kernel, dim3((uint32_t)((nq + 255) / 256)), dim3(256), 0, st, d_ts, (uint64_t)n,
                       d_win_start, d_win_end, (uint32_t)nq, d_lo, d_hi);
    GRAB_HIP(hipGetLastError());
    return GRAB_OK;
}

int sample_window_seeds_async(const uint64_t* d_sorted_ts, const uint32_t* d_ids_by_ts, size_t n,
                              const uint64_t* d_win_start, const uint64_t* d_win_end, uint64_t win_start,
                              uint64_t win_end, int per_query_window, size_t num_queries, uint32_t n_seeds,
                              uint64_t seed, uint32_t* d_out_seeds, hipStream_t st) {
    GRAB_REQUIRE(d_sorted_ts && d_ids_by_ts && d_out_seeds, "null pointer");
    GRAB_REQUIRE(!per_query_window || (d_win_start && d_win_end), "per-query windows missing");
    if (num_queries == 0 || n_seeds == 0) return GRAB_OK;
    hipLaunchKernelGGL(sample_window_seeds_kernel, dim3((uint32_t)num_queries), dim3(256), 0, st, d_sorted_ts, d_ids_by_ts,
                       (uint64_t)n, d_win_start, d_win_end, win_start, win_end, per_query_window, (uint32_t)num_queries,
                       n_seeds, seed, d_out_seeds);
    GRAB_HIP(hipGetLastError());
    return GRAB_OK;
}

}  // namespace grab

extern "C" int grab_windows_to_id_ranges(const uint64_t* d_ts, size_t n, const uint64_t* d_win_start,
                                         const uint64_t* d_win_end, size_t num_queries, uint64_t* d_lo, uint64_t* d_hi,
                                         void* stream) {
    hipStream_t st = static_cast<hipStream_t>(stream);
    return grab::windows_to_id_ranges_async(d_ts, n, d_win_start, d_win_end, num_queries, d_lo, d_hi, st);
}

extern "C" int grab_sample_window_seeds(const uint64_t* d_sorted_ts, const uint32_t* d_ids_by_ts, size_t n,
                                        const uint64_t* d_win_start, const uint64_t* d_win_end, uint64_t win_start,
                                        uint64_t win_end, int per_query_window, size_t num_queries, uint32_t n_seeds,
                                        uint64_t seed, uint32_t* d_out_seeds, void* stream) {
    hipStream_t st = static_cast<hipStream_t>(stream);
    GRAB_TRY(grab::sample_window_seeds_async(d_sorted_ts, d_ids_by_ts, n, d_win_start, d_win_end, win_start, win_end,
                                             per_query_window, num_queries, n_seeds, seed, d_out_seeds, st));
    return GRAB_OK;
}

extern "C" int grab_neighbor_timestamps(const uint32_t* d_graph, const uint64_t* d_ts, size_t num_dataset, uint32_t graph_degree,
                                        uint64_t* d_out, void* stream) {
    GRAB_REQUIRE(d_graph && d_ts && d_out, "null pointer");
    const uint64_t total = (uint64_t)num_dataset * graph_degree;
    if (total == 0) return GRAB_OK;
    GRAB_REQUIRE((total + 255) / 256 < (1ull << 31), "graph too large");
    hipLaunchKernelGGL(grab::neighbor_timestamps_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), d_graph, d_ts, total, (uint64_t)num_dataset, d_out);
    GRAB_HIP(hipGetLastError());
    return GRAB_OK;
}

extern "C" int grab_neighbor_ranks(const uint32_t* d_graph, const uint32_t* d_rank, size_t num_dataset, uint32_t graph_degree,
                                   uint32_t* d_out, void* stream) {
    GRAB_REQUIRE(d_graph && d_rank && d_out, "null pointer");
    const uint64_t total = (uint64_t)num_dataset * graph_degree;
    if (total == 0) return GRAB_OK;
    GRAB_REQUIRE((total + 255) / 256 < (1ull << 31), "graph too large");
    hipLaunchKernelGGL(grab::neighbor_ranks_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), d_graph, d_rank, total, (uint64_t)num_dataset, d_out);
    GRAB_HIP(hipGetLastError());
    return GRAB_OK;
}
