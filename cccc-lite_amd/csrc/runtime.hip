#include "runtime.h"
#include "../../include/cccc_hip_quant.h"
#include <atomic>
#include <cstdio>

namespace ccq
{

static std::atomic<hipStream_t> g_stream{ nullptr };
static std::atomic<int> g_sync{ 0 };
static thread_local const char* g_last_kernel = "";

hipStream_t stream() { return g_stream.load(std::memory_order_relaxed); }
bool sync_enabled() { return g_sync.load(std::memory_order_relaxed) != 0; }
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

}    // namespace ccq

int hip_quant_set_sync(int enabled)
{
    return ccq::g_sync.exchange(enabled ? 1 : 0, std::memory_order_relaxed);
}

int hip_quant_set_stream(void* s)
{
    ccq::g_stream.store((hipStream_t)s, std::memory_order_relaxed);
    return 0;
}

const char* hip_quant_last_kernel(void) { return ccq::g_last_kernel; }
