// Floor measurements of the benchmark (bench.py --workload floor and the floor_us column of its sweeps): what a launch
// costs on this GPU when it does nothing, and when it does nothing but stream its bytes.  Built into libcccc_bench.so,
// which only bench.py loads; the product libraries do not carry these kernels.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace
{

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

// Reads `n16` 16-byte pieces with streaming (non-temporal) 128-bit loads and folds them into one dword per wave so that
// nothing is optimised away: the memory side of a weight-streaming GEMV without its arithmetic, activations or
// reduction.  A wave reads KiB-sized pieces (64 lanes x 16 bytes, one load instruction each), U per trip; PIPE: the U
// loads of the next trip are issued before the current ones are consumed (2 U in flight -- more is not always faster:
// at 48-96 MiB the plain loop wins).  CONTIG false: piece p belongs to
// wave p % waves, so all waves sweep through the buffer side by side; true: every workgroup owns one contiguous range
// whose pieces its four waves take in turn, so the requests in flight spread over the whole buffer (5-10 % faster on
// 48-96 MiB on this part).
template <int U, bool CONTIG, bool PIPE>
__global__ __launch_bounds__(256) void floor_read_kernel(const u32x4* __restrict__ src, size_t n16, uint32_t* __restrict__ sink)
{
    const size_t lane = threadIdx.x & 63;
    const size_t wave = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6), n_waves = (size_t)gridDim.x * 4;
    const size_t n_pieces = n16 / 64;                   // whole KiB pieces; the tail goes to lane-strided loads below
    // pieces of this wave: first + i * step for i < count
    size_t first, step, count;
    if constexpr (CONTIG)
    {
        const size_t begin = n_pieces * blockIdx.x / gridDim.x, end = n_pieces * (blockIdx.x + 1) / gridDim.x;
        first = begin + (threadIdx.x >> 6);
        step = 4;
        count = first < end ? (end - first + 3) / 4 : 0;
    }
    else
    {
        first = wave;
        step = n_waves;
        count = first < n_pieces ? (n_pieces - first + n_waves - 1) / n_waves : 0;
    }
    const size_t trips = (count + U - 1) / U;
    u32x4 acc = { 0u, 0u, 0u, 0u };
    auto issue = [&](size_t trip, u32x4 (&buf)[U]) {
#pragma unroll
        for (int u = 0; u < U; u++)
        {
            const size_t i = trip * U + u;
            buf[u] = u32x4{ 0u, 0u, 0u, 0u };
            if (i < count) { buf[u] = __builtin_nontemporal_load(src + (first + i * step) * 64 + lane); }
        }
    };
    auto fold = [&](const u32x4 (&buf)[U]) {
#pragma unroll
        for (int u = 0; u < U; u++) { acc ^= buf[u]; }
    };
    u32x4 a[U], b[U];
    if constexpr (PIPE)
    {
        if (trips > 0) { issue(0, a); }
        for (size_t t = 0; t < trips; t += 2)
        {
            if (t + 1 < trips) { issue(t + 1, b); }
            fold(a);
            if (t + 2 < trips) { issue(t + 2, a); }
            if (t + 1 < trips) { fold(b); }
        }
    }
    else
    {
        for (size_t t = 0; t < trips; t++)
        {
            issue(t, a);
            fold(a);
        }
    }
    for (size_t i = n_pieces * 64 + wave * 64 + lane; i < n16; i += n_waves * 64) { acc ^= src[i]; }
    uint32_t v = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) { v ^= __shfl_xor(v, off, 64); }
    if (lane == 0) { sink[wave & 4095] = v; }
}

// One wave that reads one dword and writes it back: a launch with a single dependent trip to memory.
__global__ void touch_kernel(uint32_t* p) { if (threadIdx.x == 0) { p[0] = p[1] + 1u; } }

__global__ void empty_kernel() {}

struct Events
{
    hipEvent_t e0 = nullptr, e1 = nullptr;
    bool ok;
    Events() { ok = hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess; }
    ~Events()
    {
        if (e0) { (void)hipEventDestroy(e0); }
        if (e1) { (void)hipEventDestroy(e1); }
    }
};

}    // namespace

extern "C" {

// Average microseconds per launch of the streaming-read kernel over `iters` launches that rotate through `n_bufs`
// distinct buffers of `bytes` each (as the GEMV sweeps rotate their weights), after `warmup` launches.
// wgs_per_cu workgroups of 256 threads per compute unit (capped by the work); contiguous != 0: every workgroup reads one
// contiguous range instead of pieces at a grid stride; pipelined != 0: eight KiB pieces in flight per wave instead of four.
// Negative on error.
double cccc_bench_floor_read(int n_bufs, void** bufs, unsigned long long bytes, int wgs_per_cu, int iters, int warmup, int contiguous, int pipelined)
{
    if (n_bufs <= 0 || !bufs || bytes < 16 || iters <= 0) { return -1.0; }
    Events ev;
    if (!ev.ok) { return -1.0; }
    hipDeviceProp_t prop;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) { return -2.0; }
    uint32_t* sink = nullptr;
    if (hipMalloc(&sink, 4096 * sizeof(uint32_t)) != hipSuccess) { return -3.0; }
    const size_t n16 = bytes / 16;
    size_t grid = (n16 + 2047) / 2048;                   // at least two KiB pieces per wave
    const size_t cap = (size_t)prop.multiProcessorCount * (wgs_per_cu > 0 ? wgs_per_cu : 8);
    if (grid > cap) { grid = cap; }
    for (int i = 0; i < warmup + iters; i++)
    {
        if (i == warmup) { (void)hipEventRecord(ev.e0, nullptr); }
        const u32x4* src = (const u32x4*)bufs[i % n_bufs];
        if (contiguous && pipelined) { floor_read_kernel<4, true, true><<<(unsigned)grid, 256, 0, nullptr>>>(src, n16, sink); }
        else if (contiguous) { floor_read_kernel<4, true, false><<<(unsigned)grid, 256, 0, nullptr>>>(src, n16, sink); }
        else if (pipelined) { floor_read_kernel<4, false, true><<<(unsigned)grid, 256, 0, nullptr>>>(src, n16, sink); }
        else { floor_read_kernel<4, false, false><<<(unsigned)grid, 256, 0, nullptr>>>(src, n16, sink); }
    }
    (void)hipEventRecord(ev.e1, nullptr);
    double result = -4.0;
    if (hipEventSynchronize(ev.e1) == hipSuccess && hipGetLastError() == hipSuccess)
    {
        float ms = 0;
        (void)hipEventElapsedTime(&ms, ev.e0, ev.e1);
        result = (double)ms * 1000.0 / iters;
    }
    (void)hipFree(sink);
    return result;
}

// Average microseconds per launch of `n_launches` dependent launches (one stream, in order) replayed as one hipGraph
// `reps` times: kind 0 = empty kernel, 1 = one wave with one dependent trip to memory.  Negative on error.
double cccc_bench_launch_us(int n_launches, int reps, int kind)
{
    if (n_launches <= 0 || reps <= 0) { return -1.0; }
    Events ev;
    if (!ev.ok) { return -1.0; }
    hipStream_t stream = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    uint32_t* cell = nullptr;
    if (hipMalloc(&cell, 256) != hipSuccess) { return -3.0; }
    if (hipStreamCreate(&stream) != hipSuccess)
    {
        (void)hipFree(cell);
        return -4.0;
    }
    bool ok = hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal) == hipSuccess;
    for (int i = 0; ok && i < n_launches; i++)
    {
        if (kind == 0) { empty_kernel<<<1, 64, 0, stream>>>(); }
        else { touch_kernel<<<1, 64, 0, stream>>>(cell); }
    }
    ok = (hipStreamEndCapture(stream, &graph) == hipSuccess) && ok;
    if (ok) { ok = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0) == hipSuccess; }
    if (ok) { ok = hipGraphLaunch(exec, stream) == hipSuccess && hipStreamSynchronize(stream) == hipSuccess; }
    double result = -5.0;
    if (ok)
    {
        (void)hipEventRecord(ev.e0, stream);
        for (int r = 0; r < reps; r++) { ok = (hipGraphLaunch(exec, stream) == hipSuccess) && ok; }
        (void)hipEventRecord(ev.e1, stream);
        ok = (hipEventSynchronize(ev.e1) == hipSuccess) && ok;
        if (ok)
        {
            float ms = 0;
            (void)hipEventElapsedTime(&ms, ev.e0, ev.e1);
            result = (double)ms * 1000.0 / ((double)reps * n_launches);
        }
    }
    if (exec) { (void)hipGraphExecDestroy(exec); }
    if (graph) { (void)hipGraphDestroy(graph); }
    (void)hipStreamDestroy(stream);
    (void)hipFree(cell);
    return result;
}

}    // extern "C"
