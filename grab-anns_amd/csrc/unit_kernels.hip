// Single-purpose kernels that expose the device building blocks one by one (host pointers
// in, host pointers out), so that each can be checked against its CPU model the way the
// reference checks its own (tests/test_bitonic.cu, tests/test_sort_impl.cu,
// tests/test_hashmap.cu).  Also the small device-memory helpers of the C ABI.
#include <algorithm>
#include <vector>

#include "common.hpp"
#include "device_utils.hpp"

namespace grab {
using namespace dev;
namespace {

// one wave sorts up to 64*NPL (key,val) pairs; missing elements are padded with the largest key
template <int NPL>
__global__ void __launch_bounds__(64) sort_pairs_kernel(float* keys, uint32_t* vals, uint32_t n) {
    const int lane = threadIdx.x;
    uint64_t k[NPL];
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
        const uint32_t g = lane * NPL + i;
        k[i] = g < n ? make_sel_key(keys[g], vals[g]) : kInvalidKey;
    }
    wave_bitonic_sort<NPL>(k);
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
        const uint32_t g = lane * NPL + i;
        if (g < n) {
            keys[g] = ord_float((uint32_t)(k[i] >> 32));
            vals[g] = (uint32_t)(k[i] & 0xFFFFFFFFull);
        }
    }
}

// mirrors test_hashmap_kernel of tests/test_hashmap.cu:20-55: 256 threads insert concurrently
__global__ void __launch_bounds__(256) hash_insert_kernel(uint32_t bitlen, uint32_t n, const uint32_t* keys,
                                                          uint32_t* results, uint32_t* table_out) {
    extern __shared__ uint32_t table[];
    const uint32_t size = 1u << bitlen;
    for (uint32_t i = threadIdx.x; i < size; i += blockDim.x) table[i] = kInvalidId;
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) results[i] = hash_insert(table, bitlen, keys[i]) == 1 ? 1u : 0u;
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < size; i += blockDim.x) table_out[i] = table[i];
}

template <int METRIC>
__global__ void __launch_bounds__(256) distance_many_kernel(const float* q, const float* data, uint32_t dim,
                                                            const uint32_t* ids, uint32_t n, float* out) {
    const uint32_t g = (blockIdx.x * 256 + threadIdx.x) >> 3;
    const int j = threadIdx.x & 7;
    if (g >= n) return;  // uniform per group of 8 lanes
    const float d = group8_distance<METRIC>(q, data + (size_t)ids[g] * dim, dim, j);
    if (j == 0) out[g] = d;
}

// plain copy, 16 bytes per thread per step: the yardstick for memory-traffic counters
__global__ void __launch_bounds__(256) copy_kernel(const float4* __restrict__ src, float4* __restrict__ dst, size_t n16) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (size_t)gridDim.x * 256) dst[i] = src[i];
}

}  // namespace

int device_copy_async(void* dst, const void* src, size_t bytes, hipStream_t stream, uint32_t max_groups) {
    GRAB_REQUIRE(bytes % 16 == 0 && ((uintptr_t)dst | (uintptr_t)src) % 16 == 0, "copy of %zu bytes: size and pointers must be multiples of 16", bytes);
    if (bytes == 0) return GRAB_OK;
    const size_t n16 = bytes / 16;
    const uint32_t grid = (uint32_t)std::min<size_t>((n16 + 255) / 256, max_groups ? max_groups : 65536);
    hipLaunchKernelGGL(copy_kernel, dim3(grid), dim3(256), 0, stream, static_cast<const float4*>(src), static_cast<float4*>(dst), n16);
    GRAB_HIP(hipGetLastError());
    return GRAB_OK;
}

}  // namespace grab

using namespace grab;

extern "C" {

int grab_sort_pairs(float* keys, uint32_t* vals, size_t n) {
    GRAB_REQUIRE(keys && vals, "null pointer");
    GRAB_REQUIRE(n <= 1024, "at most 1024 pairs");
    if (n == 0) return GRAB_OK;
    DeviceScratch dk, dv;
    GRAB_HIP(dk.alloc(n * 4));
    GRAB_HIP(dv.alloc(n * 4));
    GRAB_HIP(hipMemcpy(dk.ptr, keys, n * 4, hipMemcpyHostToDevice));
    GRAB_HIP(hipMemcpy(dv.ptr, vals, n * 4, hipMemcpyHostToDevice));
    const uint32_t nn = (uint32_t)n;
    if (n <= 64) hipLaunchKernelGGL(sort_pairs_kernel<1>, dim3(1), dim3(64), 0, 0, dk.as<float>(), dv.as<uint32_t>(), nn);
    else if (n <= 128) hipLaunchKernelGGL(sort_pairs_kernel<2>, dim3(1), dim3(64), 0, 0, dk.as<float>(), dv.as<uint32_t>(), nn);
    else if (n <= 256) hipLaunchKernelGGL(sort_pairs_kernel<4>, dim3(1), dim3(64), 0, 0, dk.as<float>(), dv.as<uint32_t>(), nn);
    else if (n <= 512) hipLaunchKernelGGL(sort_pairs_kernel<8>, dim3(1), dim3(64), 0, 0, dk.as<float>(), dv.as<uint32_t>(), nn);
    else hipLaunchKernelGGL(sort_pairs_kernel<16>, dim3(1), dim3(64), 0, 0, dk.as<float>(), dv.as<uint32_t>(), nn);
    GRAB_HIP(hipGetLastError());
    GRAB_HIP(hipMemcpy(keys, dk.ptr, n * 4, hipMemcpyDeviceToHost));
    GRAB_HIP(hipMemcpy(vals, dv.ptr, n * 4, hipMemcpyDeviceToHost));
    return GRAB_OK;
}

int grab_hash_insert_many(uint32_t bitlen, const uint32_t* keys, size_t n, uint32_t* results,
                          uint32_t* table_out) {
    GRAB_REQUIRE(keys && results && table_out, "null pointer");
    GRAB_REQUIRE(bitlen >= 1 && bitlen <= 15, "bitlen must be in [1,15] for the LDS table");
    const size_t size = (size_t)1 << bitlen;
    DeviceScratch dk, dr, dt;
    GRAB_HIP(dk.alloc(n * 4));
    GRAB_HIP(dr.alloc(n * 4));
    GRAB_HIP(dt.alloc(size * 4));
    GRAB_HIP(hipMemcpy(dk.ptr, keys, n * 4, hipMemcpyHostToDevice));
    if (size * 4 > 64 * 1024)
        GRAB_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(hash_insert_kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)(size * 4)));
    hipLaunchKernelGGL(hash_insert_kernel, dim3(1), dim3(256), size * 4, 0, bitlen, (uint32_t)n,
                       dk.as<uint32_t>(), dr.as<uint32_t>(), dt.as<uint32_t>());
    GRAB_HIP(hipGetLastError());
    GRAB_HIP(hipMemcpy(results, dr.ptr, n * 4, hipMemcpyDeviceToHost));
    GRAB_HIP(hipMemcpy(table_out, dt.ptr, size * 4, hipMemcpyDeviceToHost));
    return GRAB_OK;
}

int grab_distance_many(const float* query, const float* data, size_t num_rows, uint32_t dim,
                       const uint32_t* ids, size_t n, int metric, float* out) {
    GRAB_REQUIRE(query && data && ids && out, "null pointer");
    GRAB_REQUIRE(dim >= 4 && dim % 4 == 0, "unsupported dimension %u (must be a multiple of 4)", dim);
    for (size_t i = 0; i < n; ++i) GRAB_REQUIRE(ids[i] < num_rows, "id %u out of range", ids[i]);
    if (n == 0) return GRAB_OK;
    DeviceScratch dq, dd, di, dout;
    GRAB_HIP(dq.alloc((size_t)dim * 4));
    GRAB_HIP(dd.alloc(num_rows * dim * 4));
    GRAB_HIP(di.alloc(n * 4));
    GRAB_HIP(dout.alloc(n * 4));
    GRAB_HIP(hipMemcpy(dq.ptr, query, (size_t)dim * 4, hipMemcpyHostToDevice));
    GRAB_HIP(hipMemcpy(dd.ptr, data, num_rows * dim * 4, hipMemcpyHostToDevice));
    GRAB_HIP(hipMemcpy(di.ptr, ids, n * 4, hipMemcpyHostToDevice));
    const uint32_t blocks = (uint32_t)((n * 8 + 255) / 256);
    if (metric == GRAB_METRIC_IP)
        hipLaunchKernelGGL(distance_many_kernel<kMetricIP>, dim3(blocks), dim3(256), 0, 0, dq.as<float>(),
                           dd.as<float>(), dim, di.as<uint32_t>(), (uint32_t)n, dout.as<float>());
    else
        hipLaunchKernelGGL(distance_many_kernel<kMetricL2>, dim3(blocks), dim3(256), 0, 0, dq.as<float>(),
                           dd.as<float>(), dim, di.as<uint32_t>(), (uint32_t)n, dout.as<float>());
    GRAB_HIP(hipGetLastError());
    GRAB_HIP(hipMemcpy(out, dout.ptr, n * 4, hipMemcpyDeviceToHost));
    return GRAB_OK;
}

// ---- device memory helpers for callers without a HIP binding of their own ----
int grab_device_malloc(void** out, size_t bytes) {
    GRAB_REQUIRE(out != nullptr, "null pointer");
    GRAB_HIP(hipMalloc(out, bytes ? bytes : 1));
    return GRAB_OK;
}
int grab_device_free(void* p) {
    if (p) GRAB_HIP(hipFree(p));
    return GRAB_OK;
}
int grab_copy_to_device(void* dst, const void* src, size_t bytes) {
    GRAB_HIP(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
    return GRAB_OK;
}
int grab_copy_to_host(void* dst, const void* src, size_t bytes) {
    GRAB_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
    return GRAB_OK;
}
int grab_copy_to_device_async(void* dst, const void* src, size_t bytes, void* stream) {
    if (bytes == 0) return GRAB_OK;
    GRAB_REQUIRE(dst && src, "null pointer");
    GRAB_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, static_cast<hipStream_t>(stream)));
    return GRAB_OK;
}
int grab_copy_to_host_async(void* dst, const void* src, size_t bytes, void* stream) {
    if (bytes == 0) return GRAB_OK;
    GRAB_REQUIRE(dst && src, "null pointer");
    GRAB_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, static_cast<hipStream_t>(stream)));
    return GRAB_OK;
}
int grab_host_malloc(void** out, size_t bytes) {
    GRAB_REQUIRE(out != nullptr, "null pointer");
    GRAB_HIP(hipHostMalloc(out, bytes ? bytes : 1, hipHostMallocDefault));
    return GRAB_OK;
}
int grab_host_free(void* p) {
    if (p) GRAB_HIP(hipHostFree(p));
    return GRAB_OK;
}
int grab_device_memset(void* dst, int value, size_t bytes) {
    GRAB_HIP(hipMemset(dst, value, bytes));
    return GRAB_OK;
}
int grab_device_copy(void* dst, const void* src, size_t bytes) {
    GRAB_REQUIRE(dst && src && bytes % 16 == 0, "device copy needs non-null pointers and a multiple of 16 bytes");
    if (bytes == 0) return GRAB_OK;
    const size_t n16 = bytes / 16;
    const uint32_t grid = (uint32_t)std::min<size_t>((n16 + 255) / 256, 65536);
    hipLaunchKernelGGL(copy_kernel, dim3(grid), dim3(256), 0, 0, static_cast<const float4*>(src), static_cast<float4*>(dst), n16);
    GRAB_HIP(hipGetLastError());
    GRAB_HIP(hipDeviceSynchronize());
    return GRAB_OK;
}
int grab_device_memory(size_t* free_bytes, size_t* total_bytes) {
    size_t f = 0, t = 0;
    GRAB_HIP(hipMemGetInfo(&f, &t));
    if (free_bytes) *free_bytes = f;
    if (total_bytes) *total_bytes = t;
    return GRAB_OK;
}
int grab_device_synchronize(void) {
    GRAB_HIP(hipDeviceSynchronize());
    return GRAB_OK;
}
int grab_stream_create(void** out_stream) {
    GRAB_REQUIRE(out_stream != nullptr, "null pointer");
    hipStream_t s = nullptr;
    GRAB_HIP(hipStreamCreate(&s));
    *out_stream = s;
    return GRAB_OK;
}
int grab_stream_destroy(void* stream) {
    if (stream) GRAB_HIP(hipStreamDestroy(static_cast<hipStream_t>(stream)));
    return GRAB_OK;
}
int grab_stream_synchronize(void* stream) {
    GRAB_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    return GRAB_OK;
}
int grab_stream_wait(void* stream, void* other) {
    if (stream == other) return GRAB_OK;
    hipEvent_t ev = nullptr;
    GRAB_HIP(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
    hipError_t e = hipEventRecord(ev, static_cast<hipStream_t>(other));
    if (e == hipSuccess) e = hipStreamWaitEvent(static_cast<hipStream_t>(stream), ev, 0);
    (void)hipEventDestroy(ev);  // released by the runtime once the recorded work has completed
    GRAB_HIP(e);
    return GRAB_OK;
}

}  // extern "C"
