// Growable device buffer on HIP virtual memory management.
// Same contract as cagra::DeviceBufferVMM (src/vmm_allocator.cuh:23-118): reserve the address
// range once, map one more physical allocation at the tail on every growth, never shrink,
// never move.
#include <vector>

#include "common.hpp"

struct grab_vmm {
    void* base = nullptr;
    size_t capacity = 0;
    size_t mapped = 0;
    size_t granularity = 0;
    int device = 0;
    std::vector<hipMemGenericAllocationHandle_t> handles;
    std::vector<size_t> handle_bytes;
};

using namespace grab;

namespace {
hipMemAllocationProp device_prop(int device) {
    hipMemAllocationProp prop = {};
    prop.type = hipMemAllocationTypePinned;
    prop.location.type = hipMemLocationTypeDevice;
    prop.location.id = device;
    return prop;
}
}  // namespace

extern "C" {

int grab_vmm_create(size_t max_capacity_bytes, grab_vmm** out) {
    GRAB_REQUIRE(out != nullptr, "null output pointer");
    GRAB_REQUIRE(max_capacity_bytes > 0, "capacity must be positive");
    auto* b = new grab_vmm();
    hipError_t e = hipGetDevice(&b->device);
    hipMemAllocationProp prop = device_prop(b->device);
    // The reference asks for the minimum granularity (2 MiB on its hardware).  HIP reports
    // 4 KiB here; growth steps are rounded to 2 MiB so that a buffer is made of few mappings.
    if (e == hipSuccess) e = hipMemGetAllocationGranularity(&b->granularity, &prop, hipMemAllocationGranularityRecommended);
    if (e == hipSuccess && b->granularity < (2u << 20)) b->granularity = 2u << 20;
    if (e == hipSuccess) {
        b->capacity = (max_capacity_bytes + b->granularity - 1) / b->granularity * b->granularity;
        e = hipMemAddressReserve(&b->base, b->capacity, 0, nullptr, 0);
    }
    if (e != hipSuccess) {
        set_error("HIP error %s while reserving %zu bytes of address space", hipGetErrorString(e), max_capacity_bytes);
        delete b;
        return GRAB_ERR_HIP;
    }
    *out = b;
    return GRAB_OK;
}

int grab_vmm_resize(grab_vmm* b, size_t new_size) {
    GRAB_REQUIRE(b != nullptr, "null buffer");
    if (new_size <= b->mapped) return GRAB_OK;  // vmm_allocator.cuh:71
    if (new_size > b->capacity) {               // vmm_allocator.cuh:72-74
        set_error("VMM OOM: Request exceeds reserved capacity (%zu > %zu)", new_size, b->capacity);
        return GRAB_ERR_CAPACITY;
    }
    const size_t aligned = (new_size + b->granularity - 1) / b->granularity * b->granularity;
    const size_t diff = aligned - b->mapped;
    if (diff == 0) return GRAB_OK;
    hipMemAllocationProp prop = device_prop(b->device);
    hipMemGenericAllocationHandle_t handle;
    GRAB_HIP(hipMemCreate(&handle, diff, &prop, 0));
    char* at = static_cast<char*>(b->base) + b->mapped;
    const char* what = "hipMemMap";
    hipError_t e = hipMemMap(at, diff, 0, handle, 0);
    if (e == hipSuccess) {
        hipMemAccessDesc desc = {};
        desc.location.type = hipMemLocationTypeDevice;
        desc.location.id = b->device;
        desc.flags = hipMemAccessFlagsProtReadWrite;
        what = "hipMemSetAccess";
        // access is (re)declared for the whole mapped prefix: on this runtime hipMemSetAccess on
        // the new sub-range alone is rejected once an earlier mapping of a different size exists
        e = hipMemSetAccess(b->base, b->mapped + diff, &desc, 1);
        if (e != hipSuccess) (void)hipMemUnmap(at, diff);
    }
    if (e != hipSuccess) {
        (void)hipMemRelease(handle);
        set_error("HIP error %s in %s of %zu bytes at offset %zu (granularity %zu)", hipGetErrorString(e), what, diff,
                  b->mapped, b->granularity);
        return GRAB_ERR_HIP;
    }
    b->handles.push_back(handle);
    b->handle_bytes.push_back(diff);
    b->mapped = aligned;
    return GRAB_OK;
}

void* grab_vmm_data(const grab_vmm* b) { return b ? b->base : nullptr; }
size_t grab_vmm_size(const grab_vmm* b) { return b ? b->mapped : 0; }
size_t grab_vmm_capacity(const grab_vmm* b) { return b ? b->capacity : 0; }

void grab_vmm_destroy(grab_vmm* b) {
    if (!b) return;
    if (b->base) {
        size_t off = 0;
        for (size_t i = 0; i < b->handles.size(); ++i) {
            (void)hipMemUnmap(static_cast<char*>(b->base) + off, b->handle_bytes[i]);
            (void)hipMemRelease(b->handles[i]);
            off += b->handle_bytes[i];
        }
        (void)hipMemAddressFree(b->base, b->capacity);
    }
    delete b;
}

}  // extern "C"
