// Ascending sort of 64-bit keys in device memory (power-of-two length, padded by the caller
// with the largest key).  Used where the reference calls thrust::sort_by_key
// (src/index/insert.cu:422-424) and for ordering queries by their window.
#include "device_sort.hpp"

namespace grab {
namespace {

constexpr uint32_t kLdsSortMax = 16384;  // 128 KB of LDS

// one workgroup, bitonic network in LDS
__global__ void __launch_bounds__(1024) sort_lds_kernel(uint64_t* keys, uint32_t padded) {
    extern __shared__ uint64_t sk[];
    for (uint32_t i = threadIdx.x; i < padded; i += 1024) sk[i] = keys[i];
    __syncthreads();
    for (uint32_t size = 2; size <= padded; size <<= 1) {
        for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
            for (uint32_t t = threadIdx.x; t < padded / 2; t += 1024) {
                const uint32_t lo = ((t & ~(stride - 1)) << 1) | (t & (stride - 1)), hi = lo | stride;
                const bool up = (lo & size) == 0;
                const uint64_t a = sk[lo], b = sk[hi];
                if ((a > b) == up) {
                    sk[lo] = b;
                    sk[hi] = a;
                }
            }
            __syncthreads();
        }
    }
    for (uint32_t i = threadIdx.x; i < padded; i += 1024) keys[i] = sk[i];
}

// larger inputs: one launch per compare-exchange stage
__global__ void __launch_bounds__(256) sort_global_stage_kernel(uint64_t* keys, uint32_t padded, uint32_t size, uint32_t stride) {
    const uint32_t t = blockIdx.x * 256 + threadIdx.x;
    if (t >= padded / 2) return;
    const uint32_t lo = ((t & ~(stride - 1)) << 1) | (t & (stride - 1)), hi = lo | stride;
    const bool up = (lo & size) == 0;
    const uint64_t a = keys[lo], b = keys[hi];
    if ((a > b) == up) {
        keys[lo] = b;
        keys[hi] = a;
    }
}

// Sort by rank counting, for the few thousand keys of one insert step: a key's place is the number of keys ordered
// before it (smaller, or equal with a lower index), counted by sixteen lanes that each take every sixteenth key from
// a copy of the input in LDS.  No barrier after the copy, one launch, every CU at work - where the bitonic network of
// one workgroup spends a barrier per stage.
constexpr uint32_t kRankSortMax = 16384;  // 128 KB of LDS
constexpr uint32_t kRankLanes = 16;

__global__ void __launch_bounds__(256) rank_sort_kernel(const uint64_t* __restrict__ in, uint64_t* __restrict__ out, uint32_t n) {
    extern __shared__ uint64_t sk[];
    for (uint32_t i = threadIdx.x; i < n; i += 256) sk[i] = in[i];
    __syncthreads();
    const uint32_t i = blockIdx.x * (256 / kRankLanes) + threadIdx.x / kRankLanes, s = threadIdx.x % kRankLanes;
    const uint64_t mine = i < n ? sk[i] : ~0ull;
    uint32_t cnt = 0, j = s;
    for (; j + 7 * kRankLanes < n; j += 8 * kRankLanes) {
        uint64_t v[8];
#pragma unroll
        for (uint32_t u = 0; u < 8; ++u) v[u] = sk[j + u * kRankLanes];
#pragma unroll
        for (uint32_t u = 0; u < 8; ++u) cnt += (v[u] < mine || (v[u] == mine && j + u * kRankLanes < i)) ? 1u : 0u;
    }
    for (; j < n; j += kRankLanes) {
        const uint64_t v = sk[j];
        cnt += (v < mine || (v == mine && j < i)) ? 1u : 0u;
    }
#pragma unroll
    for (int m = 1; m < (int)kRankLanes; m <<= 1) cnt += __shfl_xor(cnt, m, 64);
    if (s == 0 && i < n) out[cnt] = mine;
}

}  // namespace

int rank_sort_u64_async(const uint64_t* d_in, uint64_t* d_out, uint32_t n, hipStream_t st) {
    GRAB_REQUIRE(d_in != nullptr && d_out != nullptr && d_in != d_out, "rank sort needs two distinct buffers");
    if (n == 0) return GRAB_OK;
    if (n > kRankSortMax) {
        GRAB_HIP(hipMemcpyAsync(d_out, d_in, (size_t)n * sizeof(uint64_t), hipMemcpyDeviceToDevice, st));
        return sort_u64_async(d_out, n, st);
    }
    const size_t lds = (size_t)n * sizeof(uint64_t);
    if (lds > 64 * 1024)
        GRAB_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(rank_sort_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds));
    hipLaunchKernelGGL(rank_sort_kernel, dim3((n + 256 / kRankLanes - 1) / (256 / kRankLanes)), dim3(256), lds, st, d_in, d_out, n);
    GRAB_HIP(hipGetLastError());
    return GRAB_OK;
}

int sort_u64_async(uint64_t* d_keys, uint32_t padded, hipStream_t st) {
    GRAB_REQUIRE(d_keys != nullptr, "null keys");
    GRAB_REQUIRE(padded >= 2 && (padded & (padded - 1)) == 0, "sort length must be a power of two");
    if (padded <= kLdsSortMax) {
        const size_t lds = (size_t)padded * sizeof(uint64_t);
        if (lds > 64 * 1024)
            GRAB_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(sort_lds_kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        hipLaunchKernelGGL(sort_lds_kernel, dim3(1), dim3(1024), lds, st, d_keys, padded);
    } else {
        for (uint32_t size = 2; size <= padded; size <<= 1)
            for (uint32_t stride = size >> 1; stride > 0; stride >>= 1)
                hipLaunchKernelGGL(sort_global_stage_kernel, dim3((padded / 2 + 255) / 256), dim3(256), 0, st, d_keys, padded, size, stride);
    }
    GRAB_HIP(hipGetLastError());
    return GRAB_OK;
}

}  // namespace grab
