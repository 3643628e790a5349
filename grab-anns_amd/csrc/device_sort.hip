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

}  // namespace

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
