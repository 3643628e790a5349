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

// keys sk[s + 16 m], m in [m0, m1), that are smaller than `mine` (OR_EQUAL: or equal to it)
template <bool OR_EQUAL>
__device__ __forceinline__ uint32_t rank_count(const uint64_t* sk, uint32_t s, uint32_t m0, uint32_t m1, uint64_t mine) {
    uint32_t cnt = 0, m = m0;
    for (; m + 8 <= m1; m += 8) {
        uint64_t v[8];
#pragma unroll
        for (uint32_t u = 0; u < 8; ++u) v[u] = sk[s + (m + u) * kRankLanes];
#pragma unroll
        for (uint32_t u = 0; u < 8; ++u) cnt += (OR_EQUAL ? v[u] <= mine : v[u] < mine) ? 1u : 0u;
    }
    for (; m < m1; ++m) {
        const uint64_t v = sk[s + m * kRankLanes];
        cnt += (OR_EQUAL ? v <= mine : v < mine) ? 1u : 0u;
    }
    return cnt;
}

__global__ void __launch_bounds__(256) rank_sort_kernel(const uint64_t* __restrict__ in, uint64_t* __restrict__ out, uint32_t n) {
    extern __shared__ uint64_t sk[];
    for (uint32_t i = threadIdx.x; i < n; i += 256) sk[i] = in[i];
    __syncthreads();
    const uint32_t i = blockIdx.x * (256 / kRankLanes) + threadIdx.x / kRankLanes, s = threadIdx.x % kRankLanes;
    const uint64_t mine = i < n ? sk[i] : ~0ull;
    // an equal key goes first when its index is lower: "<=" for the keys before position i, "<" from there on
    const uint32_t m_end = n > s ? (n - s + kRankLanes - 1) / kRankLanes : 0;                     // keys of this lane
    const uint32_t m_mid = i > s ? min((i - s + kRankLanes - 1) / kRankLanes, m_end) : 0;         // those below i
    uint32_t cnt = rank_count<true>(sk, s, 0, m_mid, mine) + rank_count<false>(sk, s, m_mid, m_end, mine);
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
