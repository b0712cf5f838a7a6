// HIP-only device control of the host mirror: what the reference's GpuControl does for this path
// (cccc/GpuControl.h:115-121 per-device BLAS handle, cccc/GpuControl.cpp:18 thread_local current
// device, :311-327 setAsCurrent, :459-516 tracked malloc/free).
#pragma once
#include "Rocblas.h"
#include <cstddef>
#include <map>
#include <memory>
#include <mutex>

namespace cccc
{

class GpuControl
{
public:
    explicit GpuControl(int device_id);
    ~GpuControl();
    GpuControl(const GpuControl&) = delete;
    GpuControl& operator=(const GpuControl&) = delete;

    // One GpuControl per device id, created on first use.
    static GpuControl* select(int device_id);
    static GpuControl* getCurrentGpu();

    int getDeviceId() const { return device_id_; }
    void setAsCurrent();

    // Tracked allocations: every pointer handed out is remembered with its size so that free()
    // of a foreign pointer is refused and leaks can be counted.
    int malloc(void** p, size_t bytes);
    int free(void* p);
    size_t allocatedBytes() const;

    static int copyHostToDevice(void* dst, const void* src, size_t bytes);
    static int copyDeviceToHost(void* dst, const void* src, size_t bytes);
    static int copyDeviceToDevice(void* dst, const void* src, size_t bytes);

    Rocblas* rocblas_ = nullptr;

private:
    int device_id_ = 0;
    mutable std::mutex mutex_;
    std::map<void*, size_t> malloc_map_;
    std::unique_ptr<Rocblas> rocblas_owner_;
};

}    // namespace cccc
