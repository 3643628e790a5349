// cagra::DeviceBufferVMM with the reference's interface (src/vmm_allocator.cuh:23-118) over the C ABI.
#pragma once
#include <cstddef>
#include <stdexcept>
#include <string>

#include "grab_anns.h"

namespace cagra {

class DeviceBufferVMM {
public:
    explicit DeviceBufferVMM(size_t max_capacity_bytes) {
        if (grab_vmm_create(max_capacity_bytes, &buf_) != GRAB_OK) throw std::runtime_error(grab_last_error());
    }
    ~DeviceBufferVMM() { free(); }
    DeviceBufferVMM(const DeviceBufferVMM&) = delete;
    DeviceBufferVMM& operator=(const DeviceBufferVMM&) = delete;

    void free() {
        grab_vmm_destroy(buf_);
        buf_ = nullptr;
    }
    // no-op when new_size <= size(); throws "VMM OOM: ..." past the reserved capacity (:70-74)
    void resize(size_t new_size) {
        if (grab_vmm_resize(buf_, new_size) != GRAB_OK) throw std::runtime_error(grab_last_error());
    }
    void* data() const { return grab_vmm_data(buf_); }
    size_t size() const { return grab_vmm_size(buf_); }

private:
    grab_vmm* buf_ = nullptr;
};

}  // namespace cagra
