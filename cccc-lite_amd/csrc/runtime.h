// Host-side state shared by the entry points: the stream work is enqueued on, the
// synchronise-after-launch switch, and the error convention of the reference's HIP library
// (cccc-hip/hip_functions.cpp:32-42: 0 ok, 1 runtime error with a message on stderr).
#pragma once
#include <hip/hip_runtime.h>

namespace ccq
{

hipStream_t stream();
bool sync_enabled();
void note_kernel(const char* name);

// Called after every launch: picks up launch errors, and when the sync switch is on also waits
// for the device like the reference does after each kernel.
int finish(const char* what);

// Number of compute units of the current device (cached per device).
int cu_count();

// Device scratch memory of at least `bytes` for the launches about to be enqueued on `stream()`: one
// grow-only buffer per (host thread, device, stream), kept until the process ends, so kernels this thread
// enqueues on one stream reuse it in order and no other thread can replace it under them.  Returns nullptr when it cannot be provided (allocation failure, or the buffer would
// have to grow while the stream is being captured into a graph); callers then take a path that needs none.
void* workspace(size_t bytes);

// Where a k-split GEMM keeps its FP32 partial sums.  Default (no SplitScratch, or strict == false): workspace()
// above.  strict: the fixed buffer and nothing else, so nothing is ever allocated -- a request beyond
// fixed_bytes (or with no buffer at all) is recorded in `refused` and the caller reports an error instead of
// launching.
struct SplitScratch
{
    bool strict = false;
    float* fixed = nullptr;
    size_t fixed_bytes = 0;
    size_t refused = 0;
};

// The load-time tiled copy registered for the FP8 weight `W` by hip_quant_weight_prepare, or nullptr
// when there is none or its type / shape / row stride differ (defined with the registry in dispatch.hip).
const unsigned char* lookup_tiled(const void* W, int type, int n_out, int K, long long ldw);

}    // namespace ccq
