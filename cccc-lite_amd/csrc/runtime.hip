#include "runtime.h"
#include "../../include/cccc_hip_quant.h"
#include <atomic>
#include <cstdio>
#include <map>
#include <utility>

namespace ccq
{

// Per host thread, like the reference's current-device pointer (cccc/GpuControl.cpp:18): one thread
// capturing its launches into a graph on its own stream does not redirect another thread's work.
static thread_local hipStream_t g_stream = nullptr;
static thread_local int g_sync = 0;
static thread_local const char* g_last_kernel = "";

hipStream_t stream() { return g_stream; }
bool sync_enabled() { return g_sync != 0; }
void note_kernel(const char* name) { g_last_kernel = name; }

int finish(const char* what)
{
    hipError_t err = hipGetLastError();
    if (err == hipSuccess && sync_enabled()) { err = hipDeviceSynchronize(); }
    if (err != hipSuccess)
    {
        fprintf(stderr, "%s kernel launch failed: %s\n", what, hipGetErrorString(err));
        return 1;
    }
    return 0;
}

int cu_count()
{
    constexpr int kMaxDevices = 64;
    static std::atomic<int> cached[kMaxDevices];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) { return 256; }
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n == 0)
    {
        hipDeviceProp_t prop;
        n = (hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0) ? prop.multiProcessorCount : 256;
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

// One grow-only buffer per (host thread, device, stream).  A buffer is only ever replaced by the thread that uses it,
// after that thread has waited for the stream, so the pointer handed out stays valid until the same thread asks again:
// no other thread can free it between this call and the launch that follows.  Two host threads that enqueue on one
// stream each get a buffer of their own.
void* workspace(size_t bytes)
{
    struct Buffer { void* ptr; size_t bytes; };
    static thread_local std::map<std::pair<int, hipStream_t>, Buffer> buffers;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) { return nullptr; }
    Buffer& b = buffers[{ dev, stream() }];
    if (b.bytes >= bytes) { return b.ptr; }
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream(), &capture) != hipSuccess || capture != hipStreamCaptureStatusNone)
    {
        (void)hipGetLastError();
        return nullptr;
    }
    // this thread's earlier launches on the stream may still be using the old buffer
    if (b.ptr && (hipStreamSynchronize(stream()) != hipSuccess || hipFree(b.ptr) != hipSuccess)) { (void)hipGetLastError(); }
    b = Buffer{ nullptr, 0 };
    const size_t want = bytes + bytes / 4;
    void* p = nullptr;
    if (hipMalloc(&p, want) != hipSuccess)
    {
        (void)hipGetLastError();
        return nullptr;
    }
    b = Buffer{ p, want };
    return p;
}

}    // namespace ccq

int hip_quant_set_sync(int enabled)
{
    const int before = ccq::g_sync;
    ccq::g_sync = enabled ? 1 : 0;
    return before;
}

int hip_quant_set_stream(void* s)
{
    ccq::g_stream = (hipStream_t)s;
    return 0;
}

int hip_quant_workspace_reserve(unsigned long long bytes)
{
    if (bytes == 0) { return 0; }
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(ccq::stream(), &capture) != hipSuccess || capture != hipStreamCaptureStatusNone)
    {
        (void)hipGetLastError();
        return -1;
    }
    return ccq::workspace((size_t)bytes) ? 0 : 1;
}

void* hip_quant_get_stream(void) { return (void*)ccq::g_stream; }

const char* hip_quant_last_kernel(void) { return ccq::g_last_kernel; }
