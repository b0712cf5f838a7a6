// Timing loops of the benchmark, in native code because Python call overhead would dominate microsecond
// kernels.  Built into libcccc_bench.so, which only bench.py loads; the host library does not carry them.
#include "DecodeModel.h"
#include "Matrix.h"
#include "../../include/cccc_hip_quant.h"
#include <hip/hip_runtime.h>
#include <cstdio>
#include <vector>

using namespace cccc;

namespace
{

// Two timing events and the library's sync switch (off while timing), both put back on every way out.
struct TimingScope
{
    hipEvent_t e0 = nullptr, e1 = nullptr;
    int previous_sync;
    bool ok;
    TimingScope() : previous_sync(hip_quant_set_sync(0))
    {
        ok = hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess;
    }
    ~TimingScope()
    {
        if (e0) { (void)hipEventDestroy(e0); }
        if (e1) { (void)hipEventDestroy(e1); }
        hip_quant_set_sync(previous_sync);
    }
    TimingScope(const TimingScope&) = delete;
    TimingScope& operator=(const TimingScope&) = delete;
};

}    // namespace

extern "C" {

// Runs `steps` timed passes over a chain of n_ops linears  R[i] = W[i]^T X[i]  (Matrix::mulBatched
// with TRANS / NO_TRANS, as the LLM graph calls it) after `warmup` untimed passes.  use_graph != 0
// replays one captured hipGraph per pass instead of issuing the launches one by one.  Events are
// recorded on the stream the kernels run on.  Returns elapsed milliseconds for all timed passes, or
// a negative value on error.
double cccc_bench_linear_chain(int n_ops, void** W, void** X, void** R, int steps, int warmup, int use_graph)
{
    auto one_pass = [&]() -> int {
        int status = 0;
        for (int i = 0; i < n_ops; i++)
        {
            const int rc = Matrix::mulBatched(*(Matrix*)W[i], *(Matrix*)X[i], *(Matrix*)R[i], MATRIX_TRANS, MATRIX_NO_TRANS, 1.0f, 0.0f);
            if (rc != 0) { status = rc; }
        }
        return status;
    };
    hipStream_t stream = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    TimingScope timing;
    if (!timing.ok) { return -1.0; }
    const hipEvent_t e0 = timing.e0, e1 = timing.e1;
    double result = -1.0;
    for (int i = 0; i < warmup; i++) { if (one_pass() != 0) { return -2.0; } }
    if (hipDeviceSynchronize() != hipSuccess) { return -3.0; }
    if (use_graph)
    {
        if (hipStreamCreate(&stream) != hipSuccess) { return -4.0; }
        hip_quant_set_stream(stream);
        bool ok = hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal) == hipSuccess;
        if (ok) { ok = one_pass() == 0; }
        ok = (hipStreamEndCapture(stream, &graph) == hipSuccess) && ok;
        hip_quant_set_stream(nullptr);
        if (ok) { ok = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0) == hipSuccess; }
        if (ok) { ok = hipGraphLaunch(exec, stream) == hipSuccess && hipStreamSynchronize(stream) == hipSuccess; }
        if (ok)
        {
            (void)hipEventRecord(e0, stream);
            for (int s = 0; s < steps; s++) { (void)hipGraphLaunch(exec, stream); }
            (void)hipEventRecord(e1, stream);
            ok = hipEventSynchronize(e1) == hipSuccess;
        }
        if (ok)
        {
            float ms = 0;
            (void)hipEventElapsedTime(&ms, e0, e1);
            result = ms;
        }
        if (exec) { (void)hipGraphExecDestroy(exec); }
        if (graph) { (void)hipGraphDestroy(graph); }
        (void)hipStreamDestroy(stream);
    }
    else
    {
        (void)hipEventRecord(e0, nullptr);
        bool ok = true;
        for (int s = 0; s < steps; s++) { ok = (one_pass() == 0) && ok; }
        (void)hipEventRecord(e1, nullptr);
        ok = (hipEventSynchronize(e1) == hipSuccess) && ok;
        if (ok)
        {
            float ms = 0;
            (void)hipEventElapsedTime(&ms, e0, e1);
            result = ms;
        }
    }
    return result;
}

// Times `iters` back-to-back FP4 block-scale linears  Y = W[i % n_w]^T X  issued straight through
// hip_quant_gemm (the host mirror always passes the reference's block size 16; this loop lets the
// benchmark also measure block 32).  Returns elapsed milliseconds or a negative value on error.
double cccc_bench_fp4_chain(int n_w, void** W, void** S, void* X, void* Y, int n_out, int tokens, int K,
                            unsigned int block, int iters, int warmup)
{
    TimingScope timing;
    if (!timing.ok) { return -1.0; }
    const hipEvent_t e0 = timing.e0, e1 = timing.e1;
    int status = 0;
    for (int i = 0; i < warmup + iters; i++)
    {
        if (i == warmup) { (void)hipEventRecord(e0, nullptr); }
        const int rc = hip_quant_gemm(1, 0, n_out, tokens, K, 1.0f, W[i % n_w], (int)FP4_E2M1, K, 1.0f, X, (int)BFLOAT16, K, 1.0f,
                                      0.0f, Y, (int)BFLOAT16, n_out, 0.0f, S[i % n_w], nullptr, block);
        if (rc != 0) { status = rc; }
    }
    (void)hipEventRecord(e1, nullptr);
    double result = -2.0;
    if (hipEventSynchronize(e1) == hipSuccess && status == 0)
    {
        float ms = 0;
        (void)hipEventElapsedTime(&ms, e0, e1);
        result = ms;
    }
    return result;
}

// Times `reps` passes over every layer's fused gate/up launch of a DecodeModel (RMSNorm + SwiGLU pair, distinct
// weights per layer), the pass captured once and replayed as a hipGraph the way the decode step runs, with events on the
// launch stream; returns the average microseconds per launch or < 0.
double cccc_decode_bench_gate_up(void* model, int reps)
{
    DecodeModel* m = (DecodeModel*)model;
    const DecodeConfig& cfg = m->config();
    if (reps <= 0 || cfg.layers <= 0) { return -2.0; }
    TimingScope timing;
    if (!timing.ok) { return -1.0; }
    auto one_pass = [&]() -> bool {
        bool ok = true;
        for (int li = 0; li < cfg.layers; li++)
        {
            Matrix *gate = m->tensor(li, DecodeModel::W_GATE), *up = m->tensor(li, DecodeModel::W_UP);
            hip_fused_linear gu{};
            gu.w_type = (int)gate->getDataType();
            gu.K = cfg.hidden;
            gu.n_segments = 2;
            gu.pair = 1;
            gu.W[0] = gate->data(); gu.n_out[0] = cfg.inter; gu.w_scale[0] = gate->getQuantScale();
            gu.W[1] = up->data(); gu.n_out[1] = cfg.inter; gu.w_scale[1] = up->getQuantScale();
            gu.Y[0] = m->activation(DecodeModel::ACT_GATED)->data();
            gu.X = m->activation(DecodeModel::ACT_R1)->data();
            gu.norm_weight = m->tensor(li, DecodeModel::RMS_FFN)->data();
            gu.norm_eps = cfg.eps;
            ok = (hip_quant_linear_fused(&gu) == 0) && ok;
        }
        return ok;
    };
    if (!one_pass() || hipDeviceSynchronize() != hipSuccess) { return -3.0; }          // warm-up
    hipStream_t stream = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    if (hipStreamCreate(&stream) != hipSuccess) { return -4.0; }
    hip_quant_set_stream(stream);
    bool ok = hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal) == hipSuccess;
    if (ok) { ok = one_pass(); }
    ok = (hipStreamEndCapture(stream, &graph) == hipSuccess) && ok;
    hip_quant_set_stream(nullptr);
    if (ok) { ok = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0) == hipSuccess; }
    if (ok) { ok = hipGraphLaunch(exec, stream) == hipSuccess && hipStreamSynchronize(stream) == hipSuccess; }
    float ms = 0;
    if (ok)
    {
        (void)hipEventRecord(timing.e0, stream);
        for (int rep = 0; rep < reps; rep++) { (void)hipGraphLaunch(exec, stream); }
        (void)hipEventRecord(timing.e1, stream);
        ok = hipEventSynchronize(timing.e1) == hipSuccess;
    }
    if (ok) { (void)hipEventElapsedTime(&ms, timing.e0, timing.e1); }
    if (exec) { (void)hipGraphExecDestroy(exec); }
    if (graph) { (void)hipGraphDestroy(graph); }
    (void)hipStreamDestroy(stream);
    return ok ? (double)ms * 1000.0 / ((double)reps * cfg.layers) : -3.0;
}

}    // extern "C"
