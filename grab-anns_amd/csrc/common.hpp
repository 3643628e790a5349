// Shared host-side helpers of the library: status codes, error text, HIP call checking.
#pragma once
#include <algorithm>
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>

#include "grab_anns.h"

namespace grab {

void set_error(const char* fmt, ...);
const char* get_error();

// A failed HIP call becomes GRAB_ERR_HIP with the call site in the error text.  The reference
// prints and exits (CUDA_CHECK, src/index/cagra.cuh:9-17); a library must not.
#define GRAB_HIP(call)                                                                     \
    do {                                                                                   \
        hipError_t e__ = (call);                                                           \
        if (e__ != hipSuccess) {                                                           \
            ::grab::set_error("HIP error %s at %s:%d: %s", hipGetErrorString(e__), __FILE__, \
                              __LINE__, #call);                                            \
            return GRAB_ERR_HIP;                                                           \
        }                                                                                  \
    } while (0)

#define GRAB_REQUIRE(cond, ...)            \
    do {                                   \
        if (!(cond)) {                     \
            ::grab::set_error(__VA_ARGS__); \
            return GRAB_ERR_INVALID;       \
        }                                  \
    } while (0)

#define GRAB_TRY(expr)              \
    do {                            \
        int rc__ = (expr);          \
        if (rc__ != GRAB_OK) return rc__; \
    } while (0)

inline uint64_t splitmix64(uint64_t* state) {
    uint64_t z = (*state += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

// Device scratch that is freed on scope exit (stateless entry points allocate per call, as
// the reference's wrappers do).
// A caller that runs the same allocating routine many times in a row (the buckets of the time-partitioned graph: a
// dozen allocations and frees per bucket, each a wait for the device) can lend the calling thread one block of device
// memory: while an arena is set, DeviceScratch takes its memory from it, bump-allocated, and gives nothing back; the
// caller rewinds it between runs.  What does not fit is allocated as ever.  `wanted` adds up what was asked for.
struct ScratchArena {
    char* base = nullptr;
    size_t cap = 0, used = 0, wanted = 0;
};
ScratchArena*& scratch_arena();  // of the calling thread; null by default

struct DeviceScratch {
    void* ptr = nullptr;
    bool owned = true;
    ~DeviceScratch() {
        if (ptr && owned) (void)hipFree(ptr);
    }
    hipError_t alloc(size_t bytes) {
        if (ScratchArena* a = scratch_arena()) {
            const size_t need = (std::max<size_t>(bytes, 1) + 255) & ~(size_t)255;
            a->wanted += need;
            if (a->used + need <= a->cap) {
                ptr = a->base + a->used;
                a->used += need;
                owned = false;
                return hipSuccess;
            }
        }
        return hipMalloc(&ptr, bytes ? bytes : 1);
    }
    template <class T>
    T* as() const {
        return static_cast<T*>(ptr);
    }
};

// plain copy by a kernel on `stream`, 16 bytes per thread per step (unit_kernels.hip).  Either side may be page-locked
// host memory: the copy then stays on the stream's compute queue, with no hand-over to a copy engine and back.
// bytes must be a multiple of 16, both pointers 16-byte aligned.
// max_groups > 0: at most that many workgroups walk the buffer (a copy that waits on a host link needs few of the device's
// wave slots, and leaves the rest to the kernels it runs beside).
int device_copy_async(void* dst, const void* src, size_t bytes, hipStream_t stream, uint32_t max_groups = 0);

}  // namespace grab
