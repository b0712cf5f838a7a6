// Neighbours of the quantized linear inside one batch-1 decode step of a Qwen3-style transformer,
// gfx950, BF16 activations.  Every kernel keeps the reference's rounding points -- each op of the
// reference graph writes a BF16 tensor with FP32 math inside:
//   RMSNorm   y = bf16(x * invstd * w), invstd = rsqrtf(sum(x^2) / n + eps)    cccc-hip/hip_functions.cpp:1506-1535
//   RoPE      half-rotate, tables BF16, rotation in FP32                        cccc-hip/hip_functions.cpp:1719-1738
//   attention scores = bf16(scale * K^T q); softmax in FP32 -> BF16 probabilities; y = bf16(V p)
//             cccc/MatrixEx.cpp:3018-3104, cccc-hip/hip_functions.cpp:776-804 (softmax), :2225-2239 (mask)
//   SiLU      bf16(x * bf16(sigmoid(x))), product bf16(s * u)                    cccc/MatrixEx.cpp:756-762,
//             cccc-hip/hip_functions.cpp:722-732, :953-966
//   residual  bf16(a + b)                                                       cccc-hip/hip_functions.cpp:895-908
// Where the reference runs ~45 one-thread-per-element launches per layer (with a device sync after
// each), these are fused around the GEMVs: the step position and the current token live in device
// memory so that a whole step is a fixed launch sequence (replayable as one hipGraph).
#pragma once
#include "gemv_kernels.h"

namespace ccq
{

__device__ __forceinline__ float bf16_round(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }

// (value, index) order of the greedy pick: larger value first, lower index on ties; NaN never wins
__device__ __forceinline__ bool better(float v, unsigned i, float bv, unsigned bi) { return v > bv || (v == bv && i < bi); }

// best (value, index) over the 64 lanes of a wave, in every lane
__device__ __forceinline__ void wave_argmax(float& bv, unsigned& bi)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1)
    {
        const float ov = __shfl_xor(bv, off);
        const unsigned oi = __shfl_xor(bi, off);
        if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
    }
}

// Candidate list a linear kernel leaves for the greedy pick (optional, single-segment launches): one
// (value, index) per wave or workgroup of the launch.  Layout: [0] count, [4..15] unused, then `capacity` floats,
// then `capacity` indices, capacity = n_out / 2 + 16 (no launch shape has more waves than row pairs plus one workgroup).
struct ArgmaxCandidates
{
    unsigned* count;
    float* value;
    unsigned* index;
};

__host__ __device__ __forceinline__ ArgmaxCandidates argmax_candidates(void* workspace, unsigned n)
{
    const unsigned capacity = n / 2u + 16u;
    ArgmaxCandidates c;
    c.count = (unsigned*)workspace;
    c.value = (float*)((char*)workspace + 16);
    c.index = (unsigned*)((char*)workspace + 16 + (size_t)capacity * 4);
    return c;
}

// Sum over a workgroup of THREADS threads; every thread gets the result.  `scratch` holds THREADS / 64 floats.
template <int THREADS>
__device__ __forceinline__ float block_sum(float v, float* scratch)
{
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0) { scratch[threadIdx.x >> 6] = v; }
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int w = 0; w < THREADS / 64; w++) { total += scratch[w]; }
    __syncthreads();
    return total;
}

// ------------------------------------------------------------------------------------------
// Fused decode GEMV (one token):  x' = [rmsnorm](x);  y_s = W_s x'  for up to three weight segments
// sharing x' (q / k / v), or the SwiGLU pair  y = bf16(silu(W_0 x') * (W_1 x'));  optional residual.

struct FusedLinearArgs
{
    const uint8_t* W[3];
    uint16_t* Y[3];
    int n_out[3];
    float w_scale[3];
    int n_segments;
    int pair;                  // 1: SwiGLU pair of W[0] (gate) and W[1] (up) into Y[0]
    int K;
    const uint16_t* X;         // bf16 [K]
    const uint16_t* norm_w;    // bf16 [K] or nullptr
    float norm_eps;
    const uint16_t* residual;  // bf16 [n_out[0]] or nullptr (single segment / pair only)
    const uint8_t* T[3];       // load-time tiled copies of W[s] (matrix-core variant only)
    const uint8_t* S[3];       // FP4 only: E4M3 block scales of W[s], one byte per `block` elements of the flat index
    unsigned block;            // FP4 only: 16 or 32
    void* argmax_ws;           // single segment only: candidate list of the outputs for the greedy pick, or nullptr
};

// Staging of the activation vector into LDS in the [step][half][lane] layout of the dot2 kernels,
// with RMSNorm on the way when asked, in two parts so that the caller can put its first weight
// requests between them: vector-memory loads complete in issue order, so a wait for the activation
// would otherwise also wait for every weight request issued before it.  The first PRE 16-byte
// chunks of each thread travel in registers; longer vectors take the slower loop in finish().
constexpr int STAGE_PRE = 4;

struct StagedActivation
{
    u32x4 x[STAGE_PRE], w[STAGE_PRE];
};

// PARTS 16-byte pieces per lane and k-step: 2 for FP8 rows (a step is 1024 codes), 4 for FP4 rows (2048 codes)
template <int PARTS = 2>
__device__ __forceinline__ int stage_slot(int c)
{
    const int step = c / (64 * PARTS), in_step = c % (64 * PARTS);
    return (step * PARTS + (in_step % PARTS)) * 64 + in_step / PARTS;
}

template <int THREADS>
__device__ __forceinline__ void stage_issue(const FusedLinearArgs& a, StagedActivation& r)
{
#pragma unroll
    for (int j = 0; j < STAGE_PRE; j++)
    {
        const int c = threadIdx.x + j * THREADS;
        r.x[j] = r.w[j] = u32x4{ 0u, 0u, 0u, 0u };
        if (c * 8 < a.K)
        {
            r.x[j] = *(const u32x4*)(a.X + c * 8);
            if (a.norm_w) { r.w[j] = *(const u32x4*)(a.norm_w + c * 8); }
        }
    }
}

// `red` holds THREADS / 64 floats.  Ends with a barrier: xs is complete for every thread.
template <int THREADS, int PARTS = 2>
__device__ __forceinline__ void stage_finish(const FusedLinearArgs& a, const StagedActivation& r, u32x4* xs, float* red)
{
    const int n_steps = (a.K + 512 * PARTS - 1) / (512 * PARTS);
    const int n_chunks = n_steps * 64 * PARTS;               // 16-byte chunks incl. zero padding
    float sumsq = 0.0f;
    if (a.norm_w)
    {
#pragma unroll
        for (int j = 0; j < STAGE_PRE; j++) { sumsq += sumsq8(r.x[j]); }
    }
    else
    {
#pragma unroll
        for (int j = 0; j < STAGE_PRE; j++)
        {
            const int c = threadIdx.x + j * THREADS;
            if (c < n_chunks) { xs[stage_slot<PARTS>(c)] = r.x[j]; }
        }
    }
    for (int c = threadIdx.x + STAGE_PRE * THREADS; c < n_chunks; c += THREADS)
    {
        u32x4 v = { 0u, 0u, 0u, 0u };
        if (c * 8 < a.K) { v = *(const u32x4*)(a.X + c * 8); }
        if (a.norm_w) { sumsq += sumsq8(v); }
        xs[stage_slot<PARTS>(c)] = v;
    }
    if (a.norm_w)
    {
        // block sum in the order of block_sum(), without its closing barrier: `red` is not written again
        // before the barrier at the end of this function.  The barrier also publishes the raw tail chunks.
        sumsq = wave_sum(sumsq);
        if ((threadIdx.x & 63) == 0) { red[threadIdx.x >> 6] = sumsq; }
        __syncthreads();
        float total = 0.0f;
#pragma unroll
        for (int w = 0; w < THREADS / 64; w++) { total += red[w]; }
        const float invstd = rsqrtf(total / (float)a.K + a.norm_eps);
#pragma unroll
        for (int j = 0; j < STAGE_PRE; j++)
        {
            const int c = threadIdx.x + j * THREADS;
            if (c < n_chunks) { xs[stage_slot<PARTS>(c)] = normed8(r.x[j], r.w[j], invstd); }    // padding chunks are zero
        }
        for (int c = threadIdx.x + STAGE_PRE * THREADS; c < n_chunks; c += THREADS)
        {
            if (c * 8 < a.K) { xs[stage_slot<PARTS>(c)] = normed8(xs[stage_slot<PARTS>(c)], *(const u32x4*)(a.norm_w + c * 8), invstd); }
        }
    }
    __syncthreads();
}

// What one lane does with the two finished sums of a row group: the SwiGLU pair bf16(silu(gate) * up) with the
// reference's three roundings (group g = output g), or two plain outputs; the residual is added to a rounded value.
__device__ __forceinline__ void store_candidate(const FusedLinearArgs& a, unsigned slot, unsigned n_slots, float v, unsigned i)
{
    const ArgmaxCandidates c = argmax_candidates(a.argmax_ws, (unsigned)a.n_out[0]);
    c.value[slot] = v;
    c.index[slot] = i;
    if (slot == 0) { *c.count = n_slots; }
}

__device__ __forceinline__ void fused_store(const FusedLinearArgs& a, int g, int seg, int row0, int row1, float t0, float t1, float& best_v, unsigned& best_i)
{
    if (a.pair)
    {
        const float gate = bf16_round(t0), up = bf16_round(t1);
        const float sig = bf16_round(1.0f / (1.0f + expf(-gate)));
        const float silu = bf16_round(gate * sig);
        float out = bf16_round(silu * up);
        if (a.residual) { out = bf16_round(out + bf16_bits_to_f32(a.residual[g])); }
        a.Y[0][g] = (uint16_t)f32_to_bf16_bits(out);
    }
    else
    {
        float o0 = bf16_round(t0), o1 = bf16_round(t1);
        if (a.residual && seg == 0)
        {
            o0 = bf16_round(o0 + bf16_bits_to_f32(a.residual[row0]));
            o1 = bf16_round(o1 + bf16_bits_to_f32(a.residual[row1]));
        }
        a.Y[seg][row0] = (uint16_t)f32_to_bf16_bits(o0);
        if (row1 != row0) { a.Y[seg][row1] = (uint16_t)f32_to_bf16_bits(o1); }
        // greedy candidates are taken on the values as stored (rounded to BF16)
        if (better(o0, (unsigned)row0, best_v, best_i)) { best_v = o0; best_i = (unsigned)row0; }
        if (better(o1, (unsigned)row1, best_v, best_i)) { best_v = o1; best_i = (unsigned)row1; }
    }
}

// One wave owns a group of two rows at a time and walks its groups in batches of U KiB per row.  The
// weights of the next batch are requested before the current one is consumed, and those of the very
// first batch before the activation is staged, so the norm prologue and every reduction overlap loads.
struct FusedRows
{
    const uint8_t *w0, *w1;
    float s0, s1;
    int seg, row0, row1;
};

// DIRECT_X (no RMSNorm in front, K a multiple of 1024): the activation is not staged at all -- every lane requests
// the 32 bytes of x it needs for a step together with the weights of that step (x is a few KiB and stays in
// the CU's L1), so the kernel has no prologue, no LDS and no barrier.
// WT == DT_BF16: the weight is not quantized at all (a tied lm_head is the embedding table, which the reference keeps in
// BF16: cccc/Net.cpp:1158-1190) -- the same kernel with 2-byte elements: a lane's 16-byte load is eight elements, a k-step
// 512 of them, and the products need no conversion.  Staged activation only.
template <int WT, int U, int WAVES, bool SCALED, bool DIRECT_X = false>
__global__ __launch_bounds__(WAVES * 64) void gemv8_fused_kernel(const FusedLinearArgs a)
{
    constexpr bool PLAIN = WT == DT_BF16;
    static_assert(!(PLAIN && (DIRECT_X || SCALED)), "BF16 weights: staged activation, no scale");
    constexpr int STEP = PLAIN ? 512 : 1024;                // elements of a row one wave-wide load covers
    constexpr int ELEM = PLAIN ? 2 : 1;                     // bytes per weight element
    constexpr int PARTS = PLAIN ? 1 : 2;                    // 16-byte activation pieces per lane and k-step
    extern __shared__ u32x4 xs[];
    __shared__ float red[WAVES];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_steps = (a.K + STEP - 1) / STEP;
    const int batches = (n_steps + U - 1) / U;
    // row groups of two: in pair mode (gate row i, up row i); otherwise two consecutive rows of one segment
    const int g0 = a.pair ? a.n_out[0] : (a.n_out[0] + 1) / 2;
    const int g1 = (a.pair || a.n_segments < 2) ? g0 : g0 + (a.n_out[1] + 1) / 2;
    const int n_groups = (a.pair || a.n_segments < 3) ? g1 : g1 + (a.n_out[2] + 1) / 2;
    const int stride = gridDim.x * WAVES;

    auto locate = [&](int g) {
        FusedRows r;
        r.seg = 0;
        if (a.pair) { r.row0 = r.row1 = g; }
        else
        {
            int local = g;
            if (g >= g1) { r.seg = 2; local = g - g1; }
            else if (g >= g0) { r.seg = 1; local = g - g0; }
            r.row0 = local * 2;
            r.row1 = min(local * 2 + 1, a.n_out[r.seg] - 1);
        }
        const int sa = a.pair ? 0 : r.seg, sb = a.pair ? 1 : r.seg;
        r.w0 = a.W[sa] + (long long)r.row0 * a.K * ELEM;
        r.w1 = a.W[sb] + (long long)r.row1 * a.K * ELEM;
        r.s0 = a.w_scale[sa];
        r.s1 = a.w_scale[sb];
        return r;
    };
    u32x4 xa[DIRECT_X ? U : 1][2], xn[DIRECT_X ? U : 1][2];      // x of the current / next batch (DIRECT_X)
    auto request = [&](const FusedRows& r, int st0, u32x4* wa, u32x4* wb, u32x4 (*xq)[2]) {
#pragma unroll
        for (int u = 0; u < U; u++)
        {
            wa[u] = wb[u] = u32x4{ 0u, 0u, 0u, 0u };
            const int k = (st0 + u) * STEP + lane * (16 / ELEM);
            if (k < a.K)
            {
                if constexpr (DIRECT_X)
                {
                    xq[u][0] = *(const u32x4*)(a.X + k);
                    xq[u][1] = *(const u32x4*)(a.X + k + 8);
                }
                wa[u] = __builtin_nontemporal_load((const u32x4*)(r.w0 + (long long)k * ELEM));
                wb[u] = __builtin_nontemporal_load((const u32x4*)(r.w1 + (long long)k * ELEM));
            }
        }
    };

    int g = blockIdx.x * WAVES + wave, batch = 0;
    FusedRows cur{}, nxt{};
    u32x4 wa[U], wb[U], na[U], nb[U];
    StagedActivation staged;
    if constexpr (!DIRECT_X) { stage_issue<WAVES * 64>(a, staged); }
    if (g < n_groups)
    {
        cur = locate(g);
        request(cur, 0, wa, wb, xa);
    }
    if constexpr (!DIRECT_X) { stage_finish<WAVES * 64, PARTS>(a, staged, xs, red); }

    float acc0 = 0.0f, acc1 = 0.0f;
    float best_v = -INFINITY;                               // greedy candidate of this wave (lane 0 keeps it)
    unsigned best_i = 0xFFFFFFFFu;
    while (g < n_groups)
    {
        int ng = g, nbatch = batch + 1;
        if (nbatch == batches)
        {
            ng = g + stride;
            nbatch = 0;
        }
        if (ng < n_groups)
        {
            nxt = nbatch == 0 ? locate(ng) : cur;
            request(nxt, nbatch * U, na, nb, xn);
        }
#pragma unroll
        for (int u = 0; u < U; u++)
        {
            const int st = batch * U + u;
            if constexpr (PLAIN)
            {
                if (st < n_steps)
                {
                    const u32x4 x0 = xs[st * 64 + lane];
#pragma unroll
                    for (int d = 0; d < 4; d++)
                    {
                        const uint32_t w0 = wa[u][d], w1 = wb[u][d];       // (a bit cast straight from the vector element reads element 0)
                        acc0 = dot2_bf16(__builtin_bit_cast(bf16x2, w0), x0[d], acc0);
                        acc1 = dot2_bf16(__builtin_bit_cast(bf16x2, w1), x0[d], acc1);
                    }
                }
            }
            else if (st < n_steps)
            {
                const u32x4 x0 = DIRECT_X ? xa[u][0] : xs[(st * 2 + 0) * 64 + lane];
                const u32x4 x1 = DIRECT_X ? xa[u][1] : xs[(st * 2 + 1) * 64 + lane];
#pragma unroll
                for (int d = 0; d < 4; d++)
                {
                    const u32x4& xv = (d < 2) ? x0 : x1;
                    bf16x2 p01, p23;
                    fp8x4_to_bf16<WT, SCALED>(wa[u][d], cur.s0, p01, p23);
                    acc0 = dot2_bf16(p01, xv[(d & 1) * 2 + 0], acc0);
                    acc0 = dot2_bf16(p23, xv[(d & 1) * 2 + 1], acc0);
                    fp8x4_to_bf16<WT, SCALED>(wb[u][d], cur.s1, p01, p23);
                    acc1 = dot2_bf16(p01, xv[(d & 1) * 2 + 0], acc1);
                    acc1 = dot2_bf16(p23, xv[(d & 1) * 2 + 1], acc1);
                }
            }
        }
        if (batch == batches - 1)
        {
            const float t0 = wave_sum(acc0), t1 = wave_sum(acc1);
            acc0 = acc1 = 0.0f;
            if (lane == 0) { fused_store(a, g, cur.seg, cur.row0, cur.row1, t0, t1, best_v, best_i); }
        }
        g = ng;
        batch = nbatch;
        cur = nxt;
#pragma unroll
        for (int u = 0; u < U; u++)
        {
            wa[u] = na[u];
            wb[u] = nb[u];
            if constexpr (DIRECT_X)
            {
                xa[u][0] = xn[u][0];
                xa[u][1] = xn[u][1];
            }
        }
    }
    if (a.argmax_ws && lane == 0) { store_candidate(a, blockIdx.x * WAVES + wave, gridDim.x * WAVES, best_v, best_i); }
}

// ------------------------------------------------------------------------------------------
// The fused one-token linear for FP4_E2M1 block-scale weights (cccc/cublas_real.h:952-955 dequantises them with
// cuda_fp4_blockscale_to_bf16, cccc-cuda/cuda_functions.cu:2926-2939): same decomposition as gemv8_fused_kernel
// -- a wave owns two rows, batches of U k-steps, the next batch requested before the current one is multiplied,
// activation (normalised on the way when asked) staged once per workgroup -- with the arithmetic of
// gemv4_dot2_kernel: a 128-bit load is 32 consecutive elements of a row, i.e. 32 / BLOCK scale blocks, and
// fp4 * e4m3 is exact in BF16, so each block's dot product is taken on the bare FP4 values and multiplied by
// its scale once.  Rows are K / 2 bytes, scales run over the flat element index; K % 32 == 0.
// Dynamic LDS: ceil(K / 2048) * 4096 bytes.
template <int BLOCK, int U, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void gemv4_fused_kernel(const FusedLinearArgs a)
{
    static_assert(BLOCK == 16 || BLOCK == 32, "block scale length");
    extern __shared__ u32x4 xs[];
    __shared__ float red[WAVES];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_steps = (a.K + 2047) / 2048;
    const int batches = (n_steps + U - 1) / U;
    const int g0 = a.pair ? a.n_out[0] : (a.n_out[0] + 1) / 2;
    const int g1 = (a.pair || a.n_segments < 2) ? g0 : g0 + (a.n_out[1] + 1) / 2;
    const int n_groups = (a.pair || a.n_segments < 3) ? g1 : g1 + (a.n_out[2] + 1) / 2;
    const int stride = gridDim.x * WAVES;

    struct Rows
    {
        const uint8_t *w0, *w1, *s0, *s1;
        int seg, row0, row1;
    };
    auto locate = [&](int g) {
        Rows r;
        r.seg = 0;
        if (a.pair) { r.row0 = r.row1 = g; }
        else
        {
            int local = g;
            if (g >= g1) { r.seg = 2; local = g - g1; }
            else if (g >= g0) { r.seg = 1; local = g - g0; }
            r.row0 = local * 2;
            r.row1 = min(local * 2 + 1, a.n_out[r.seg] - 1);
        }
        const int sa = a.pair ? 0 : r.seg, sb = a.pair ? 1 : r.seg;
        r.w0 = a.W[sa] + (((long long)r.row0 * a.K) >> 1) + lane * 16;
        r.w1 = a.W[sb] + (((long long)r.row1 * a.K) >> 1) + lane * 16;
        r.s0 = a.S[sa] + ((long long)r.row0 * a.K) / BLOCK + lane * (32 / BLOCK);
        r.s1 = a.S[sb] + ((long long)r.row1 * a.K) / BLOCK + lane * (32 / BLOCK);
        return r;
    };
    auto request = [&](const Rows& r, int st0, u32x4* wa, u32x4* wb, uint32_t* sa, uint32_t* sb) {
#pragma unroll
        for (int u = 0; u < U; u++)
        {
            wa[u] = wb[u] = u32x4{ 0u, 0u, 0u, 0u };
            sa[u] = sb[u] = 0u;
            if ((st0 + u) * 2048 + lane * 32 < a.K)
            {
                wa[u] = __builtin_nontemporal_load((const u32x4*)(r.w0 + (st0 + u) * 1024));
                wb[u] = __builtin_nontemporal_load((const u32x4*)(r.w1 + (st0 + u) * 1024));
                if (BLOCK == 16)
                {
                    sa[u] = *(const uint16_t*)(r.s0 + (st0 + u) * 128);
                    sb[u] = *(const uint16_t*)(r.s1 + (st0 + u) * 128);
                }
                else
                {
                    sa[u] = r.s0[(st0 + u) * 64];
                    sb[u] = r.s1[(st0 + u) * 64];
                }
            }
        }
    };
    // sum over the 32 elements of one load of fp4 * x per scale block, times the block's scale
    auto row_dot = [&](const u32x4& w, uint32_t sc, const u32x4 (&x)[4], float acc) {
        float part[2] = { 0.0f, 0.0f };
#pragma unroll
        for (int d = 0; d < 4; d++)
        {
            const bf16x2 q0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[d], 1.0f, 0);
            const bf16x2 q1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[d], 1.0f, 1);
            const bf16x2 q2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[d], 1.0f, 2);
            const bf16x2 q3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[d], 1.0f, 3);
            float p = part[d >> 1];
            p = dot2_bf16(q0, x[d][0], p);
            p = dot2_bf16(q1, x[d][1], p);
            p = dot2_bf16(q2, x[d][2], p);
            p = dot2_bf16(q3, x[d][3], p);
            part[d >> 1] = p;
        }
        const float s_lo = e4m3_byte_to_f32(sc, 0);
        const float s_hi = BLOCK == 16 ? e4m3_byte_to_f32(sc, 1) : s_lo;
        return fmaf(s_hi, part[1], fmaf(s_lo, part[0], acc));
    };

    int g = blockIdx.x * WAVES + wave, batch = 0;
    Rows cur{}, nxt{};
    u32x4 wa[U], wb[U], na[U], nb[U];
    uint32_t sa[U], sb[U], nsa[U], nsb[U];
    StagedActivation staged;
    stage_issue<WAVES * 64>(a, staged);
    if (g < n_groups)
    {
        cur = locate(g);
        request(cur, 0, wa, wb, sa, sb);
    }
    stage_finish<WAVES * 64, 4>(a, staged, xs, red);

    float acc0 = 0.0f, acc1 = 0.0f;
    float best_v = -INFINITY;
    unsigned best_i = 0xFFFFFFFFu;
    while (g < n_groups)
    {
        int ng = g, nbatch = batch + 1;
        if (nbatch == batches)
        {
            ng = g + stride;
            nbatch = 0;
        }
        if (ng < n_groups)
        {
            nxt = nbatch == 0 ? locate(ng) : cur;
            request(nxt, nbatch * U, na, nb, nsa, nsb);
        }
#pragma unroll
        for (int u = 0; u < U; u++)
        {
            const int st = batch * U + u;
            if (st < n_steps)
            {
                u32x4 x[4];
#pragma unroll
                for (int p = 0; p < 4; p++) { x[p] = xs[(st * 4 + p) * 64 + lane]; }
                acc0 = row_dot(wa[u], sa[u], x, acc0);
                acc1 = row_dot(wb[u], sb[u], x, acc1);
            }
        }
        if (batch == batches - 1)
        {
            const float t0 = wave_sum(acc0), t1 = wave_sum(acc1);
            acc0 = acc1 = 0.0f;
            if (lane == 0) { fused_store(a, g, cur.seg, cur.row0, cur.row1, t0, t1, best_v, best_i); }
        }
        g = ng;
        batch = nbatch;
        cur = nxt;
#pragma unroll
        for (int u = 0; u < U; u++)
        {
            wa[u] = na[u];
            wb[u] = nb[u];
            sa[u] = nsa[u];
            sb[u] = nsb[u];
        }
    }
    if (a.argmax_ws && lane == 0) { store_candidate(a, blockIdx.x * WAVES + wave, gridDim.x * WAVES, best_v, best_i); }
}

// ------------------------------------------------------------------------------------------
// The same fused one-token linear on the matrix cores, reading the load-time tiled copies (T[s]):
// structure of gemv8_mfma_kernel -- a workgroup owns RT tiles of 16 rows, its waves split K in
// interleaved spans of 64 * U codes, every load instruction covers one contiguous KiB -- with the
// activation (normalised on the way when asked) staged once per workgroup in LDS and used as the
// single live column of the 16-column operand.  Up to three segments; a tile never straddles two
// segments (every segment's tiled copy is padded to whole tiles).  No SwiGLU pair mode.
// NORM = false: no RMSNorm in front, and then no staging either -- the lanes of the live column take
// their activation chunks straight from global memory and the kernel has no prologue at all.
// Dynamic LDS (NORM only): ceil(K / 1024) * 2048 bytes.
template <int WT, int RT, int U, int WAVES, bool SCALED, bool NORM>
__global__ __launch_bounds__(WAVES * 64) void gemv8_fused_mfma_kernel(const FusedLinearArgs a)
{
    extern __shared__ u32x4 xs[];
    __shared__ float red[WAVES];
    __shared__ float partial[WAVES][RT][16];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int i = lane & 15;
    const int g = lane >> 4;
    const int blocks_per_row = (a.K + 63) / 64;
    const int t0 = (a.n_out[0] + 15) / 16;
    const int t1 = a.n_segments < 2 ? t0 : t0 + (a.n_out[1] + 15) / 16;
    const int n_tiles = a.n_segments < 3 ? t1 : t1 + (a.n_out[2] + 15) / 16;

    const uint8_t* wtile[RT];
    float scale[RT];
#pragma unroll
    for (int rt = 0; rt < RT; rt++)
    {
        const int tile = min((int)blockIdx.x * RT + rt, n_tiles - 1);      // a clamped tile is computed and dropped
        const int seg = tile >= t1 ? 2 : (tile >= t0 ? 1 : 0);
        const int local = tile - (seg == 2 ? t1 : (seg == 1 ? t0 : 0));
        wtile[rt] = a.T[seg] + (long long)local * blocks_per_row * 1024 + lane * 16;
        scale[rt] = a.w_scale[seg];
    }
    const int span = 64 * U;
    // requests the weights of the span at kb and, without a norm, the matching activation chunks of the live column
    auto request = [&](int kb, u32x4 (*w)[RT], u32x4 (*x)[2]) {
#pragma unroll
        for (int u = 0; u < U; u++)
        {
            const bool in_k = kb + u * 64 + g * 16 < a.K;
#pragma unroll
            for (int rt = 0; rt < RT; rt++)
            {
                w[u][rt] = u32x4{ 0u, 0u, 0u, 0u };
                if (in_k) { w[u][rt] = __builtin_nontemporal_load((const u32x4*)(wtile[rt] + (long long)(kb + u * 64) * 16)); }
            }
            if constexpr (!NORM)
            {
                x[u][0] = x[u][1] = u32x4{ 0u, 0u, 0u, 0u };
                if (in_k && i == 0)
                {
                    x[u][0] = *(const u32x4*)(a.X + kb + u * 64 + g * 16);
                    x[u][1] = *(const u32x4*)(a.X + kb + u * 64 + g * 16 + 8);
                }
            }
        }
    };

    u32x4 w[U][RT], wn[U][RT], xr[U][2], xn[U][2];
    int kb = wave * span;
    if constexpr (NORM)
    {
        StagedActivation staged;
        stage_issue<WAVES * 64>(a, staged);
        if (kb < a.K) { request(kb, w, xr); }
        stage_finish<WAVES * 64>(a, staged, xs, red);
    }
    else if (kb < a.K) { request(kb, w, xr); }

    f32x4 acc[RT];
#pragma unroll
    for (int rt = 0; rt < RT; rt++) { acc[rt] = f32x4{ 0.0f, 0.0f, 0.0f, 0.0f }; }
    while (kb < a.K)
    {
        const int nk = kb + WAVES * span;
        if (nk < a.K) { request(nk, wn, xn); }
#pragma unroll
        for (int u = 0; u < U; u++)
        {
            // the activation of block b: codes 64 b + 16 g .. + 16 of lane group g are the 16-byte chunks 8 b + 2 g and + 1
            const int c = ((kb + u * 64) >> 3) + 2 * g;
            u32x4 x[2] = { u32x4{ 0u, 0u, 0u, 0u }, u32x4{ 0u, 0u, 0u, 0u } };
            if constexpr (NORM)
            {
                if (i == 0 && kb + u * 64 + g * 16 < a.K)
                {
                    x[0] = xs[stage_slot(c)];
                    x[1] = xs[stage_slot(c + 1)];
                }
            }
            else
            {
                x[0] = xr[u][0];
                x[1] = xr[u][1];
            }
#pragma unroll
            for (int rt = 0; rt < RT; rt++)
            {
#pragma unroll
                for (int h = 0; h < 2; h++)
                {
                    bf16x2 p0, p1, p2, p3;
                    fp8x4_to_bf16<WT, SCALED>(w[u][rt][2 * h], scale[rt], p0, p1);
                    fp8x4_to_bf16<WT, SCALED>(w[u][rt][2 * h + 1], scale[rt], p2, p3);
                    const bf16x8 wa = { p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1] };
                    acc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa, __builtin_bit_cast(bf16x8, x[h]), acc[rt], 0, 0, 0);
                }
            }
        }
        kb = nk;
#pragma unroll
        for (int u = 0; u < U; u++)
#pragma unroll
            for (int rt = 0; rt < RT; rt++) { w[u][rt] = wn[u][rt]; }
        if constexpr (!NORM)
        {
#pragma unroll
            for (int u = 0; u < U; u++)
            {
                xr[u][0] = xn[u][0];
                xr[u][1] = xn[u][1];
            }
        }
    }

    // D: lane (i, g) holds token column i, rows 4 g .. 4 g + 3; only column 0 is live
    if (i == 0)
    {
#pragma unroll
        for (int rt = 0; rt < RT; rt++)
#pragma unroll
            for (int c = 0; c < 4; c++) { partial[wave][rt][4 * g + c] = acc[rt][c]; }
    }
    __syncthreads();
    static_assert(RT * 16 <= 64, "the outputs of a workgroup are finished by its first wave");
    if (wave != 0) { return; }
    float best_v = -INFINITY;
    unsigned best_i = 0xFFFFFFFFu;
    {
        const int v = lane;
        const int rt = v >> 4, r = v & 15;
        const int tile = (int)blockIdx.x * RT + rt;
        const int seg = tile >= t1 ? 2 : (tile >= t0 ? 1 : 0);
        const int row = (tile - (seg == 2 ? t1 : (seg == 1 ? t0 : 0))) * 16 + r;
        if (v < RT * 16 && tile < n_tiles && row < a.n_out[seg])
        {
            float total = 0.0f;
#pragma unroll
            for (int wv = 0; wv < WAVES; wv++) { total += partial[wv][rt][r]; }
            float out = bf16_round(total);
            if (a.residual && seg == 0) { out = bf16_round(out + bf16_bits_to_f32(a.residual[row])); }
            a.Y[seg][row] = (uint16_t)f32_to_bf16_bits(out);
            best_v = out;
            best_i = (unsigned)row;
            if (!(out == out)) { best_v = -INFINITY; best_i = 0xFFFFFFFFu; }      // NaN never wins
        }
    }
    if (a.argmax_ws)
    {
        wave_argmax(best_v, best_i);
        if (lane == 0) { store_candidate(a, blockIdx.x, gridDim.x, best_v, best_i); }
    }
}

// ------------------------------------------------------------------------------------------
// Standalone neighbours with the reference's signatures (BF16)

// RMSNorm of `outer` rows of `inner` BF16 values, one wave per row while a row fits the wave's registers
// (inner <= 64 lanes x 8 values x RMS_CHUNKS), four rows per 256-thread workgroup: 128-bit loads, the row stays in
// registers between the sum of squares and the scaling, the 64-lane sum is the DPP reduction.  Used for the per-head
// norms (inner = 128) as well as whole hidden vectors up to 4096.  VEC = false: rows that are not whole 16-byte chunks
// (or misaligned pointers) take the same structure with scalar accesses.
constexpr int RMS_CHUNKS = 8;

template <bool VEC>
__global__ __launch_bounds__(256) void rms_norm_rows_kernel(const uint16_t* __restrict__ X, uint16_t* __restrict__ Y, const uint16_t* __restrict__ scale,
                                                           float* __restrict__ invstd_out, unsigned outer, unsigned inner, float eps)
{
    const unsigned lane = threadIdx.x & 63u;
    const unsigned row = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (row >= outer) { return; }
    const uint16_t* x = X + (size_t)row * inner;
    uint16_t* y = Y + (size_t)row * inner;
    float sumsq = 0.0f;
    if constexpr (VEC)
    {
        const unsigned n_chunks = inner / 8u;               // 16-byte chunks of the row; chunk c belongs to lane c % 64
        // every load is issued before the first use (a load inside a per-lane branch waits for the one before it: eight
        // memory latencies in a row on a 4096-wide row); lanes past the row's end re-read its last chunk and drop it
        u32x4 v[RMS_CHUNKS], w[RMS_CHUNKS];
        const int n_j = n_chunks <= 64u ? 1 : RMS_CHUNKS;   // short rows (the per-head norms) are one chunk per lane at most
#pragma unroll
        for (int j = 0; j < RMS_CHUNKS; j++)
        {
            if (j < n_j)
            {
                const unsigned c = min(lane + 64u * j, n_chunks - 1u);
                v[j] = *(const u32x4*)(x + c * 8u);
                w[j] = *(const u32x4*)(scale + c * 8u);
            }
        }
#pragma unroll
        for (int j = 0; j < RMS_CHUNKS; j++)
        {
            if (j >= n_j || lane + 64u * j >= n_chunks) { v[j] = u32x4{ 0u, 0u, 0u, 0u }; }
            sumsq += sumsq8(v[j]);
        }
        const float invstd = rsqrtf(wave_sum(sumsq) / (float)inner + eps);
        if (lane == 0 && invstd_out) { invstd_out[row] = invstd; }
#pragma unroll
        for (int j = 0; j < RMS_CHUNKS; j++)
        {
            const unsigned c = lane + 64u * j;
            if (j < n_j && c < n_chunks) { *(u32x4*)(y + c * 8u) = normed8(v[j], w[j], invstd); }
        }
    }
    else
    {
        for (unsigned i = lane; i < inner; i += 64u)
        {
            const float f = bf16_bits_to_f32(x[i]);
            sumsq = fmaf(f, f, sumsq);
        }
        const float invstd = rsqrtf(wave_sum(sumsq) / (float)inner + eps);
        if (lane == 0 && invstd_out) { invstd_out[row] = invstd; }
        for (unsigned i = lane; i < inner; i += 64u) { y[i] = (uint16_t)f32_to_bf16_bits(bf16_bits_to_f32(x[i]) * invstd * bf16_bits_to_f32(scale[i])); }
    }
}

// Half-rotate RoPE of B x T heads of D values: lane = (head row, group of eight rotation pairs), so the left half, the
// right half and the two table rows each arrive as one 128-bit load per lane and leave as one 128-bit store (D / 2 a
// multiple of 8, the model case D = 128: eight lanes per head row); any other D takes one pair per lane.
// Table row of head row r is (r % T) + pos_offset.
template <bool VEC>
__global__ __launch_bounds__(256) void rope_rows_kernel(const uint16_t* __restrict__ X, uint16_t* __restrict__ Y, const uint16_t* __restrict__ cos_tab,
                                                       const uint16_t* __restrict__ sin_tab, unsigned D, unsigned T, unsigned n_rows, unsigned pos_offset)
{
    const unsigned half = D / 2u;
    const unsigned per_row = VEC ? half / 8u : half;         // work items per head row
    const unsigned item = blockIdx.x * 256u + threadIdx.x;
    const unsigned r = item / per_row;
    if (r >= n_rows) { return; }
    const unsigned p = (item - r * per_row) * (VEC ? 8u : 1u);      // first pair of this item
    const uint16_t* x = X + (size_t)r * D + p;
    uint16_t* y = Y + (size_t)r * D + p;
    const size_t t = (size_t)(r % T + pos_offset) * half + p;
    if constexpr (VEC)
    {
        const u32x4 l = *(const u32x4*)x, rt = *(const u32x4*)(x + half);
        const u32x4 c = *(const u32x4*)(cos_tab + t), sn = *(const u32x4*)(sin_tab + t);
        u32x4 ol, orr;
#pragma unroll
        for (int d = 0; d < 4; d++)
        {
            uint32_t lo[2], hi[2];
#pragma unroll
            for (int h = 0; h < 2; h++)
            {
                const int sh = 16 * h;
                const float a = bf16_bits_to_f32((l[d] >> sh) & 0xFFFFu), b = bf16_bits_to_f32((rt[d] >> sh) & 0xFFFFu);
                const float cc = bf16_bits_to_f32((c[d] >> sh) & 0xFFFFu), ss = bf16_bits_to_f32((sn[d] >> sh) & 0xFFFFu);
                lo[h] = f32_to_bf16_bits(a * cc - b * ss);
                hi[h] = f32_to_bf16_bits(b * cc + a * ss);
            }
            ol[d] = lo[0] | (lo[1] << 16);
            orr[d] = hi[0] | (hi[1] << 16);
        }
        *(u32x4*)y = ol;
        *(u32x4*)(y + half) = orr;
    }
    else
    {
        const float a = bf16_bits_to_f32(x[0]), b = bf16_bits_to_f32(x[half]);
        const float cc = bf16_bits_to_f32(cos_tab[t]), ss = bf16_bits_to_f32(sin_tab[t]);
        y[0] = (uint16_t)f32_to_bf16_bits(a * cc - b * ss);
        y[half] = (uint16_t)f32_to_bf16_bits(b * cc + a * ss);
    }
}

// Rows longer than one wave's registers: a 256-thread workgroup per row, two passes over the row (the second one
// comes out of the cache), block-wide sum through LDS.
static __global__ __launch_bounds__(256) void rms_norm_long_rows_kernel(const uint16_t* __restrict__ X, uint16_t* __restrict__ Y, const uint16_t* __restrict__ scale,
                                                                float* __restrict__ invstd_out, unsigned inner, float eps)
{
    __shared__ float red[4];
    const uint16_t* x = X + (size_t)blockIdx.x * inner;
    uint16_t* y = Y + (size_t)blockIdx.x * inner;
    float sumsq = 0.0f;
    for (unsigned i = threadIdx.x; i < inner; i += 256u)
    {
        const float f = bf16_bits_to_f32(x[i]);
        sumsq = fmaf(f, f, sumsq);
    }
    const float invstd = rsqrtf(block_sum<256>(sumsq, red) / (float)inner + eps);
    if (threadIdx.x == 0 && invstd_out) { invstd_out[blockIdx.x] = invstd; }
    for (unsigned i = threadIdx.x; i < inner; i += 256u) { y[i] = (uint16_t)f32_to_bf16_bits(bf16_bits_to_f32(x[i]) * invstd * bf16_bits_to_f32(scale[i])); }
}

// Embedding row copy: Y[t] = W[(int)ids[t]] (ids are floats in the reference); `d_token`, when given,
// overrides ids with one int32 token id in device memory (the previous step's arg-max).
static __global__ __launch_bounds__(256) void embed_bf16_kernel(const float* __restrict__ ids, const int* __restrict__ d_token, const uint16_t* __restrict__ W,
                                                        uint16_t* __restrict__ Y, int D, int n_rows)
{
    const int t = blockIdx.y;
    int id = d_token ? d_token[t] : (int)ids[t];
    id = min(max(id, 0), n_rows - 1);
    for (int c = blockIdx.x * 256 + threadIdx.x; c * 8 < D; c += gridDim.x * 256)
    {
        *(u32x4*)(Y + (size_t)t * D + c * 8) = *(const u32x4*)(W + (size_t)id * D + c * 8);
    }
}

// ------------------------------------------------------------------------------------------
// Per-head q/k RMSNorm + RoPE + KV-cache append for one new token (head_dim 128).
// One wave per head: lanes 0..63 hold the rotation pairs (i, i + 64).
//   q   [n_q][128]  -> q_out [n_q][128] (normed, rotated)
//   k   [n_kv][128] -> k_cache[h][pos][128] (normed, rotated);  v -> v_cache[h][pos][128]
static __global__ __launch_bounds__(64) void qk_norm_rope_kv_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ k, const uint16_t* __restrict__ v,
                                                            const uint16_t* __restrict__ q_norm_w, const uint16_t* __restrict__ k_norm_w,
                                                            const uint16_t* __restrict__ cos_tab, const uint16_t* __restrict__ sin_tab,
                                                            uint16_t* __restrict__ q_out, uint16_t* __restrict__ k_cache, uint16_t* __restrict__ v_cache,
                                                            int n_q, int n_kv, int t_kv, const int* __restrict__ d_pos, float eps)
{
    const int head = blockIdx.x;            // 0 .. n_q + 2 n_kv - 1
    const int lane = threadIdx.x;
    const int pos = *d_pos;
    if (pos < 0 || pos >= t_kv) { return; }    // a position outside the cache appends nothing
    if (head >= n_q + n_kv)
    {
        const int h = head - n_q - n_kv;    // v: plain copy into the cache
        uint16_t* dst = v_cache + ((size_t)h * t_kv + pos) * 128;
        dst[lane] = v[h * 128 + lane];
        dst[lane + 64] = v[h * 128 + lane + 64];
        return;
    }
    const bool is_q = head < n_q;
    const int h = is_q ? head : head - n_q;
    const uint16_t* src = (is_q ? q : k) + h * 128;
    const uint16_t* nw = is_q ? q_norm_w : k_norm_w;
    const float xl = bf16_bits_to_f32(src[lane]), xr = bf16_bits_to_f32(src[lane + 64]);
    float nl = xl, nr = xr;                  // no norm weights (Llama-style heads): the projection output is rotated as it is
    if (nw)
    {
        const float invstd = rsqrtf(wave_sum(xl * xl + xr * xr) / 128.0f + eps);
        nl = bf16_round(xl * invstd * bf16_bits_to_f32(nw[lane]));
        nr = bf16_round(xr * invstd * bf16_bits_to_f32(nw[lane + 64]));
    }
    const float c = bf16_bits_to_f32(cos_tab[(size_t)pos * 64 + lane]), s = bf16_bits_to_f32(sin_tab[(size_t)pos * 64 + lane]);
    uint16_t* dst = is_q ? q_out + h * 128 : k_cache + ((size_t)h * t_kv + pos) * 128;
    dst[lane] = (uint16_t)f32_to_bf16_bits(nl * c - nr * s);
    dst[lane + 64] = (uint16_t)f32_to_bf16_bits(nr * c + nl * s);
}

// ------------------------------------------------------------------------------------------
// GQA decode attention, head_dim 128, group of G = n_q / n_kv query heads per KV head, two launches
// over blocks of ATT_KEYS cache positions (grid = (blocks, kv heads); blocks past *d_pos exit at once).
// 16 lanes share a cache row (8 dims each), a wave covers 4 rows per 1 KiB load, a workgroup 16, and
// every thread issues its ATT_ITS row loads before the first use.
constexpr int ATT_KEYS = 64;
constexpr int ATT_ITS = ATT_KEYS / 16;     // cache rows per thread

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) { v = fmaxf(v, __shfl_xor(v, off)); }
    return v;
}

__device__ __forceinline__ void unpack8_bf16(const u32x4& raw, float* f)
{
#pragma unroll
    for (int d = 0; d < 4; d++)
    {
        f[2 * d] = bf16_bits_to_f32(raw[d] & 0xFFFFu);
        f[2 * d + 1] = bf16_bits_to_f32(raw[d] >> 16);
    }
}

// Launch 1: scores[qh][t] = bf16(scale * k_t . q_qh) for t <= pos, and per block and query head the
// softmax statistics of its scores: stats[qh][block] = (max, sum of expf(s - max)).
template <int G>
__global__ __launch_bounds__(256) void attn_scores_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ k_cache, uint16_t* __restrict__ scores,
                                                         float2* __restrict__ stats, int t_kv, int n_blocks, const int* __restrict__ d_pos, float scale)
{
    __shared__ float s_lds[G][ATT_KEYS];
    const int kvh = blockIdx.y, blk = blockIdx.x;
    const int n_keys = min(max(*d_pos, 0), t_kv - 1) + 1;
    const int t0 = blk * ATT_KEYS;
    if (t0 >= n_keys) { return; }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane & 15;              // which 8 dims
    const int key_in_wave = lane >> 4;
    u32x4 raw[ATT_ITS];
#pragma unroll
    for (int it = 0; it < ATT_ITS; it++)
    {
        const int t = min(t0 + it * 16 + wave * 4 + key_in_wave, n_keys - 1);    // rows past the end repeat the last one and are discarded below
        raw[it] = __builtin_nontemporal_load((const u32x4*)(k_cache + ((size_t)kvh * t_kv + t) * 128 + sub * 8));
    }
    float qv[G][8];
#pragma unroll
    for (int gq = 0; gq < G; gq++) { unpack8_bf16(*(const u32x4*)(q + (size_t)(kvh * G + gq) * 128 + sub * 8), qv[gq]); }
#pragma unroll
    for (int it = 0; it < ATT_ITS; it++)
    {
        const int kl = it * 16 + wave * 4 + key_in_wave;
        const int t = t0 + kl;
        float kf[8];
        unpack8_bf16(raw[it], kf);
#pragma unroll
        for (int gq = 0; gq < G; gq++)
        {
            float dot = 0.0f;
#pragma unroll
            for (int d = 0; d < 8; d++) { dot = fmaf(kf[d], qv[gq][d], dot); }
            dot += dpp_f32<0xB1>(dot);
            dot += dpp_f32<0x4E>(dot);
            dot += dpp_f32<0x141>(dot);
            dot += dpp_f32<0x140>(dot);     // every lane of the 16-lane row holds the key's dot product
            if (sub == 0)
            {
                const uint32_t bits = f32_to_bf16_bits(scale * dot);
                if (t < n_keys) { scores[(size_t)(kvh * G + gq) * t_kv + t] = (uint16_t)bits; }
                s_lds[gq][kl] = t < n_keys ? bf16_bits_to_f32(bits) : -INFINITY;
            }
        }
    }
    __syncthreads();
    if (wave < G)
    {
        constexpr int PER_LANE = (ATT_KEYS + 63) / 64;
        float v[PER_LANE], m = -INFINITY, l = 0.0f;
#pragma unroll
        for (int j = 0; j < PER_LANE; j++) { m = fmaxf(m, v[j] = (lane + 64 * j < ATT_KEYS) ? s_lds[wave][lane + 64 * j] : -INFINITY); }
        m = wave_max(m);                                    // finite: the block holds at least one valid key
#pragma unroll
        for (int j = 0; j < PER_LANE; j++) { l += expf(v[j] - m); }
        l = wave_sum(l);
        if (lane == 0) { stats[(size_t)(kvh * G + wave) * n_blocks + blk] = make_float2(m, l); }
    }
}

// Launch 2: softmax over the whole row from the block statistics, probabilities
// p_t = bf16(expf(s_t - max) * (1 / sum)), this block's partial outputs partial[block][qh][128] (FP32).
// (Letting the last block to arrive add the partials needs a device-scope fence per workgroup, which
// writes back the L2 of every XCD: measured 17 us per launch against 3 us for launch 3.)
template <int G>
__global__ __launch_bounds__(256) void attn_pv_kernel(const uint16_t* __restrict__ scores, const float2* __restrict__ stats, const uint16_t* __restrict__ v_cache,
                                                     float* __restrict__ partial, int t_kv, int n_blocks, const int* __restrict__ d_pos, int n_q)
{
    __shared__ float acc_lds[16][G][128];   // [key slot in workgroup][head][dim]
    __shared__ float p_lds[G][ATT_KEYS];
    __shared__ float row_max[G], row_inv[G];
    const int kvh = blockIdx.y, blk = blockIdx.x;
    const int n_keys = min(max(*d_pos, 0), t_kv - 1) + 1;
    const int t0 = blk * ATT_KEYS;
    if (t0 >= n_keys) { return; }
    const int n_active = (n_keys + ATT_KEYS - 1) / ATT_KEYS;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane & 15, key_in_wave = lane >> 4;
    u32x4 raw[ATT_ITS];
#pragma unroll
    for (int it = 0; it < ATT_ITS; it++)
    {
        const int t = min(t0 + it * 16 + wave * 4 + key_in_wave, n_keys - 1);    // rows past the end get probability 0 below
        raw[it] = __builtin_nontemporal_load((const u32x4*)(v_cache + ((size_t)kvh * t_kv + t) * 128 + sub * 8));
    }
    if (wave < G)
    {
        const float2* st = stats + (size_t)(kvh * G + wave) * n_blocks;
        float m = -INFINITY;
        for (int i = lane; i < n_active; i += 64) { m = fmaxf(m, st[i].x); }
        m = wave_max(m);
        float l = 0.0f;
        for (int i = lane; i < n_active; i += 64) { l += st[i].y * expf(st[i].x - m); }
        l = wave_sum(l);
        if (lane == 0)
        {
            row_max[wave] = m;
            row_inv[wave] = l > 0.0f ? 1.0f / l : 0.0f;
        }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < G * ATT_KEYS; idx += 256)
    {
        const int gq = idx / ATT_KEYS, kl = idx % ATT_KEYS;
        const int t = t0 + kl;
        float p = 0.0f;
        if (t < n_keys) { p = bf16_round(expf(bf16_bits_to_f32(scores[(size_t)(kvh * G + gq) * t_kv + t]) - row_max[gq]) * row_inv[gq]); }
        p_lds[gq][kl] = p;
    }
    __syncthreads();
    float acc[G][8];
#pragma unroll
    for (int gq = 0; gq < G; gq++)
#pragma unroll
        for (int d = 0; d < 8; d++) { acc[gq][d] = 0.0f; }
#pragma unroll
    for (int it = 0; it < ATT_ITS; it++)
    {
        const int kl = it * 16 + wave * 4 + key_in_wave;
        float vf[8];
        unpack8_bf16(raw[it], vf);
#pragma unroll
        for (int gq = 0; gq < G; gq++)
        {
            const float p = p_lds[gq][kl];
#pragma unroll
            for (int d = 0; d < 8; d++) { acc[gq][d] = fmaf(p, vf[d], acc[gq][d]); }
        }
    }
    const int slot = wave * 4 + key_in_wave;
#pragma unroll
    for (int gq = 0; gq < G; gq++)
#pragma unroll
        for (int d = 0; d < 8; d++) { acc_lds[slot][gq][sub * 8 + d] = acc[gq][d]; }
    __syncthreads();
    for (int o = threadIdx.x; o < G * 128; o += 256)
    {
        const int gq = o >> 7, d = o & 127;
        float total = 0.0f;
#pragma unroll
        for (int sl = 0; sl < 16; sl++) { total += acc_lds[sl][gq][d]; }
        __builtin_nontemporal_store(total, &partial[((size_t)blk * n_q + kvh * G + gq) * 128 + d]);      // read once, by the merge kernel
    }
}

// Launch 3: y[o] = bf16(sum over the active blocks of partial[block][o]), in a fixed order: 64 outputs
// per workgroup, wave w adds blocks w, w + 4, ... and the four sums are added in wave order.
static __global__ __launch_bounds__(256) void attn_combine_kernel(const float* __restrict__ partial, uint16_t* __restrict__ y, int n_out, int t_kv,
                                                          const int* __restrict__ d_pos)
{
    __shared__ float part[4][64];
    const int n_keys = min(max(*d_pos, 0), t_kv - 1) + 1;
    const int n_active = (n_keys + ATT_KEYS - 1) / ATT_KEYS;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int o = blockIdx.x * 64 + lane;
    float total = 0.0f;
    if (o < n_out)
    {
        int s = wave;
        for (; s + 12 < n_active; s += 16)
        {
            const float a0 = partial[(size_t)s * n_out + o], a1 = partial[(size_t)(s + 4) * n_out + o];
            const float a2 = partial[(size_t)(s + 8) * n_out + o], a3 = partial[(size_t)(s + 12) * n_out + o];
            total = (((total + a0) + a1) + a2) + a3;
        }
        for (; s < n_active; s += 4) { total += partial[(size_t)s * n_out + o]; }
    }
    part[wave][lane] = total;
    __syncthreads();
    if (wave == 0 && o < n_out) { y[o] = (uint16_t)f32_to_bf16_bits(((part[0][lane] + part[1][lane]) + part[2][lane]) + part[3][lane]); }
}

// ------------------------------------------------------------------------------------------
// The same attention in two launches, with the q/k RMSNorm, RoPE and cache append folded in.
// Differences from the three-launch form above: the softmax of a block is taken against the block's
// own maximum and rescaled when the blocks are combined (the usual split-softmax identity), so the
// probabilities stay FP32 instead of being rounded to BF16 before they meet V.  Scores are still
// rounded to BF16.  Output differences against the three-launch form stay within about one BF16 ulp.
//
// Launch 1, grid (blocks, kv heads): raw q [n_q][128], k, v [n_kv][128] of the new token;
//   waves 0..G-1 normalise and rotate the G query heads of this KV head; the block holding row *d_pos
//   also normalises / rotates k, appends k and v to the caches, and uses them from LDS;
//   stats[qh][block] = (max, sum expf(s - max)), partial[block][qh][128] = sum expf(s_t - max) v_t.
struct HeadLoads
{
    uint16_t xl, xr, c, sn, wl, wr;       // lane's two elements of the head, its cos / sin, the two norm weights
};

__device__ __forceinline__ HeadLoads load_head(const uint16_t* __restrict__ src, const uint16_t* __restrict__ nw, const uint16_t* __restrict__ cos_row,
                                               const uint16_t* __restrict__ sin_row, int lane)
{
    return HeadLoads{ src[lane], src[lane + 64], cos_row[lane], sin_row[lane], nw ? nw[lane] : (uint16_t)0, nw ? nw[lane + 64] : (uint16_t)0 };
}

// normed == false (no per-head norm weights, Llama-style): the head is rotated as the projection left it
__device__ __forceinline__ void norm_rope_finish(const HeadLoads& h, bool normed, float eps, float& out_l, float& out_r)
{
    const float xl = bf16_bits_to_f32(h.xl), xr = bf16_bits_to_f32(h.xr);
    const float c = bf16_bits_to_f32(h.c), sn = bf16_bits_to_f32(h.sn);
    float nl = xl, nr = xr;
    if (normed)
    {
        const float wl = bf16_bits_to_f32(h.wl), wr = bf16_bits_to_f32(h.wr);
        const float invstd = rsqrtf(wave_sum(xl * xl + xr * xr) / 128.0f + eps);
        nl = bf16_round(xl * invstd * wl);
        nr = bf16_round(xr * invstd * wr);
    }
    out_l = bf16_round(nl * c - nr * sn);
    out_r = bf16_round(nr * c + nl * sn);
}

__device__ __forceinline__ void norm_rope_head(const uint16_t* __restrict__ src, const uint16_t* __restrict__ nw, const uint16_t* __restrict__ cos_row,
                                               const uint16_t* __restrict__ sin_row, float eps, int lane, float& out_l, float& out_r)
{
    norm_rope_finish(load_head(src, nw, cos_row, sin_row, lane), nw != nullptr, eps, out_l, out_r);
}

// SCORES_ONLY: the front half alone -- norm, rotation, append, the block's BF16 scores written to scores[qh][t] and their
// (max, sum expf(s - max)) to stats -- for the route that rounds the probabilities of the whole row to BF16 before they
// meet V (attn_pv_kernel and attn_combine_kernel follow); no value row is read here.
template <int G, bool SCORES_ONLY = false>
__global__ __launch_bounds__(256) void attn_fused_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ k, const uint16_t* __restrict__ v,
                                                        const uint16_t* __restrict__ q_norm_w, const uint16_t* __restrict__ k_norm_w,
                                                        const uint16_t* __restrict__ cos_tab, const uint16_t* __restrict__ sin_tab,
                                                        uint16_t* __restrict__ k_cache, uint16_t* __restrict__ v_cache,
                                                        float2* __restrict__ stats, float* __restrict__ partial,
                                                        int t_kv, int n_blocks, const int* __restrict__ d_pos, int n_q, float eps, float scale,
                                                        uint16_t* __restrict__ scores = nullptr)
{
    __shared__ float acc_lds[16][G][128];   // [key slot in workgroup][head][dim]
    __shared__ float s_lds[G][ATT_KEYS];    // scores, then expf(s - block max)
    static_assert(ATT_KEYS == 64, "the score stage gives each of the four waves one 16-key matrix-core tile");
    __shared__ __attribute__((aligned(16))) uint16_t q_lds[G][128];     // normalised, rotated query heads (BF16 values)
    __shared__ __attribute__((aligned(16))) uint16_t k_new[128];
    __shared__ float v_new[128];
    const int kvh = blockIdx.y, blk = blockIdx.x;
    const int pos = *d_pos;
    if (pos < 0 || pos >= t_kv) { return; }         // a position outside the cache: nothing to append, nothing to attend
    const int n_keys = pos + 1;
    const int t0 = blk * ATT_KEYS;
    if (t0 >= n_keys) { return; }
    const bool has_new = pos < t0 + ATT_KEYS;       // this block holds the row being appended
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane & 15, key_in_wave = lane >> 4;
    const uint16_t* cos_row = cos_tab + (size_t)pos * 64;
    const uint16_t* sin_row = sin_tab + (size_t)pos * 64;
    // the query head's few bytes are requested before the cache rows, and the key rows before the value rows:
    // loads return in the order they were issued
    HeadLoads hq{};
    if (wave < G) { hq = load_head(q + (size_t)(kvh * G + wave) * 128, q_norm_w, cos_row, sin_row, lane); }
    // Cache rows are read once per token: streaming (non-temporal) loads, like the weights, are worth 2.6 us per launch here.
    // Keys in the layout of the matrix-core row operand: wave w owns keys 16 w .. 16 w + 15 of the block, lane
    // (i = lane % 16, g = lane / 16) holds dims 32 c + 8 g .. + 7 of key i for c = 0..3.  Values as before: lane
    // (sub, key_in_wave) holds dims 8 sub .. + 7 of key it * 16 + wave * 4 + key_in_wave.
    u32x4 kraw[4], vraw[ATT_ITS];
    const int key_row = wave * 16 + sub;                                         // this lane's key within the block
    {
        const int t = min(t0 + key_row, n_keys - 1);                             // rows past the end, and row pos itself, are replaced or discarded below
#pragma unroll
        for (int c = 0; c < 4; c++) { kraw[c] = __builtin_nontemporal_load((const u32x4*)(k_cache + ((size_t)kvh * t_kv + t) * 128 + c * 32 + key_in_wave * 8)); }
    }
    if constexpr (!SCORES_ONLY)
    {
#pragma unroll
        for (int it = 0; it < ATT_ITS; it++)
        {
            const int t = min(t0 + it * 16 + wave * 4 + key_in_wave, n_keys - 1);
            vraw[it] = __builtin_nontemporal_load((const u32x4*)(v_cache + ((size_t)kvh * t_kv + t) * 128 + sub * 8));
        }
    }
    if (wave < G)
    {
        float l, r;
        norm_rope_finish(hq, q_norm_w != nullptr, eps, l, r);
        q_lds[wave][lane] = (uint16_t)f32_to_bf16_bits(l);
        q_lds[wave][lane + 64] = (uint16_t)f32_to_bf16_bits(r);
    }
    if (has_new && wave == 3)
    {
        float l, r;
        norm_rope_head(k + (size_t)kvh * 128, k_norm_w, cos_row, sin_row, eps, lane, l, r);
        k_new[lane] = (uint16_t)f32_to_bf16_bits(l);
        k_new[lane + 64] = (uint16_t)f32_to_bf16_bits(r);
        uint16_t* dst = k_cache + ((size_t)kvh * t_kv + pos) * 128;
        dst[lane] = (uint16_t)f32_to_bf16_bits(l);
        dst[lane + 64] = (uint16_t)f32_to_bf16_bits(r);
    }
    if (has_new && wave == 2)
    {
        const uint16_t a = v[(size_t)kvh * 128 + lane], b = v[(size_t)kvh * 128 + lane + 64];
        v_new[lane] = bf16_bits_to_f32(a);
        v_new[lane + 64] = bf16_bits_to_f32(b);
        uint16_t* dst = v_cache + ((size_t)kvh * t_kv + pos) * 128;
        dst[lane] = a;
        dst[lane + 64] = b;
    }
    __syncthreads();
    // scores[key][head] = K[16 keys x 128] . q^T[128 x heads]: four v_mfma_f32_16x16x32_bf16 per wave (the products of two
    // BF16 values are exact in FP32); columns G..15 of the head operand are zero.  D: lane holds head lane % 16, keys 4 g .. 4 g + 3.
    {
        f32x4 sc = { 0.0f, 0.0f, 0.0f, 0.0f };
#pragma unroll
        for (int c = 0; c < 4; c++)
        {
            u32x4 kc = kraw[c];
            if (t0 + key_row == pos) { kc = *(const u32x4*)&k_new[c * 32 + key_in_wave * 8]; }
            u32x4 qc = { 0u, 0u, 0u, 0u };
            if (sub < G) { qc = *(const u32x4*)&q_lds[sub][c * 32 + key_in_wave * 8]; }
            sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kc), __builtin_bit_cast(bf16x8, qc), sc, 0, 0, 0);
        }
        if (sub < G)
        {
#pragma unroll
            for (int v = 0; v < 4; v++)
            {
                const int kl = wave * 16 + key_in_wave * 4 + v;
                const float sv = bf16_round(scale * sc[v]);
                s_lds[sub][kl] = t0 + kl < n_keys ? sv : -INFINITY;
                if constexpr (SCORES_ONLY)
                {
                    if (t0 + kl < n_keys) { scores[(size_t)(kvh * G + sub) * t_kv + t0 + kl] = (uint16_t)(__builtin_bit_cast(uint32_t, sv) >> 16); }
                }
            }
        }
    }
    __syncthreads();
    if (wave < G)
    {
        constexpr int PER_LANE = (ATT_KEYS + 63) / 64;
        float v[PER_LANE], m = -INFINITY, l = 0.0f;
#pragma unroll
        for (int j = 0; j < PER_LANE; j++) { m = fmaxf(m, v[j] = (lane + 64 * j < ATT_KEYS) ? s_lds[wave][lane + 64 * j] : -INFINITY); }
        m = wave_max(m);                                    // finite: the block holds at least one valid key
#pragma unroll
        for (int j = 0; j < PER_LANE; j++)
        {
            const float e = expf(v[j] - m);
            if (lane + 64 * j < ATT_KEYS) { s_lds[wave][lane + 64 * j] = e; }
            l += e;
        }
        l = wave_sum(l);
        if (lane == 0) { stats[(size_t)(kvh * G + wave) * n_blocks + blk] = make_float2(m, l); }
    }
    if constexpr (SCORES_ONLY) { return; }
    __syncthreads();
    float acc[G][8];
#pragma unroll
    for (int gq = 0; gq < G; gq++)
#pragma unroll
        for (int d = 0; d < 8; d++) { acc[gq][d] = 0.0f; }
#pragma unroll
    for (int it = 0; it < ATT_ITS; it++)
    {
        const int kl = it * 16 + wave * 4 + key_in_wave;
        float vf[8];
        unpack8_bf16(vraw[it], vf);
        if (t0 + kl == pos)
        {
#pragma unroll
            for (int d = 0; d < 8; d++) { vf[d] = v_new[sub * 8 + d]; }
        }
        if (t0 + kl > pos)                                  // read from the row being appended, which may still hold anything (0 * NaN is NaN)
        {
#pragma unroll
            for (int d = 0; d < 8; d++) { vf[d] = 0.0f; }
        }
#pragma unroll
        for (int gq = 0; gq < G; gq++)
        {
            const float p = s_lds[gq][kl];                  // 0 for rows past the end
#pragma unroll
            for (int d = 0; d < 8; d++) { acc[gq][d] = fmaf(p, vf[d], acc[gq][d]); }
        }
    }
    const int slot = wave * 4 + key_in_wave;
#pragma unroll
    for (int gq = 0; gq < G; gq++)
#pragma unroll
        for (int d = 0; d < 8; d++) { acc_lds[slot][gq][sub * 8 + d] = acc[gq][d]; }
    __syncthreads();
    for (int o = threadIdx.x; o < G * 128; o += 256)
    {
        const int gq = o >> 7, d = o & 127;
        float total = 0.0f;
#pragma unroll
        for (int sl = 0; sl < 16; sl++) { total += acc_lds[sl][gq][d]; }
        __builtin_nontemporal_store(total, &partial[((size_t)blk * n_q + kvh * G + gq) * 128 + d]);      // read once, by the merge kernel
    }
}

// Launch 2: y[qh][d] = bf16(sum_b w_b partial[b][qh][d]), w_b = expf(max_b - max) / sum_b' l_b' expf(max_b' - max),
// in a fixed order.  64 outputs (half a head) per workgroup; n_blocks <= ATT_MAX_BLOCKS.
constexpr int ATT_MAX_BLOCKS = 1024;

// Every load of the common case is requested before anything is known -- the position, up to four (max, sum)
// pairs per thread and the partials of the first 64 blocks -- so the launch costs one trip to memory instead of
// three dependent ones (position -> statistics -> partials).  Blocks past the position hold whatever the
// workspace held before: they are masked out by select, never multiplied.
static __global__ __launch_bounds__(256) void attn_rescale_combine_kernel(const float* __restrict__ partial, const float2* __restrict__ stats, uint16_t* __restrict__ y,
                                                                  int n_out, int t_kv, int n_blocks, const int* __restrict__ d_pos)
{
    __shared__ float w_lds[ATT_MAX_BLOCKS];
    __shared__ float red[4];
    __shared__ float part[4][64];
    constexpr int PRE = 16;                              // blocks per wave requested up front (4 waves: 64 blocks)
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int qh = (blockIdx.x * 64) >> 7;
    const int o = min(blockIdx.x * 64 + lane, n_out - 1);
    const float2* st = stats + (size_t)qh * n_blocks;

    const int pos = *d_pos;
    const float2 mine = st[min(lane, n_blocks - 1)];    // every wave: block `lane` (used when no more than 64 blocks are live)
    float2 sb[ATT_MAX_BLOCKS / 256];
#pragma unroll
    for (int i = 0; i < ATT_MAX_BLOCKS / 256; i++) { sb[i] = st[min((int)threadIdx.x + i * 256, n_blocks - 1)]; }
    float pre[PRE];
#pragma unroll
    for (int j = 0; j < PRE; j++) { pre[j] = __builtin_nontemporal_load(&partial[(size_t)min(wave + 4 * j, n_blocks - 1) * n_out + o]); }

    if (pos < 0 || pos >= t_kv) { return; }
    const int n_active = pos / ATT_KEYS + 1;
    float total = 0.0f, inv;
    if (n_active <= 64)
    {
        // Up to 64 blocks: every wave holds one block's statistics per lane and works out the weights for
        // itself (the same reductions in the same order as below, whose other three wave sums are zero), so
        // nothing is exchanged before the final sum over the four waves.
        const bool live = lane < n_active;
        const float m = wave_max(live ? mine.x : -INFINITY);
        const float e = live ? expf(mine.x - m) : 0.0f;
        const float l = wave_sum(live ? mine.y * e : 0.0f);
        inv = l > 0.0f ? 1.0f / l : 0.0f;
#pragma unroll
        for (int j = 0; j < PRE; j++)
        {
            const int b = wave + 4 * j;
            const float w = __shfl(e, b);
            if (b < n_active) { total = fmaf(pre[j], w, total); }
        }
    }
    else
    {
        float m = -INFINITY;
#pragma unroll
        for (int i = 0; i < ATT_MAX_BLOCKS / 256; i++)
        {
            if ((int)threadIdx.x + i * 256 < n_active) { m = fmaxf(m, sb[i].x); }
        }
        m = wave_max(m);
        if (lane == 0) { red[wave] = m; }
        __syncthreads();
        m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        __syncthreads();
        float l = 0.0f;
#pragma unroll
        for (int i = 0; i < ATT_MAX_BLOCKS / 256; i++)
        {
            const int b = threadIdx.x + i * 256;
            if (b < n_active)
            {
                const float e = expf(sb[i].x - m);
                w_lds[b] = e;
                l += sb[i].y * e;
            }
        }
        l = block_sum<256>(l, red);                     // its barrier publishes w_lds
        inv = l > 0.0f ? 1.0f / l : 0.0f;
#pragma unroll
        for (int j = 0; j < PRE; j++) { total = fmaf(pre[j], w_lds[wave + 4 * j], total); }
        for (int b = wave + 4 * PRE; b < n_active; b += 4) { total = fmaf(partial[(size_t)b * n_out + o], w_lds[b], total); }
    }
    part[wave][lane] = total;
    __syncthreads();
    if (wave == 0 && blockIdx.x * 64 + lane < n_out) { y[o] = (uint16_t)f32_to_bf16_bits((((part[0][lane] + part[1][lane]) + part[2][lane]) + part[3][lane]) * inv); }
}

// Arg-max of BF16 values, lowest index on ties, in two launches: per-block candidates, then the pick.

template <int THREADS>
__device__ __forceinline__ void block_argmax(float& bv, unsigned& bi, float* best_v, unsigned* best_i)
{
    wave_argmax(bv, bi);
    if ((threadIdx.x & 63) == 0) { best_v[threadIdx.x >> 6] = bv; best_i[threadIdx.x >> 6] = bi; }
    __syncthreads();
    if (threadIdx.x == 0)
    {
        for (int w = 1; w < THREADS / 64; w++)
        {
            if (better(best_v[w], best_i[w], bv, bi)) { bv = best_v[w]; bi = best_i[w]; }
        }
    }
}

constexpr int ARGMAX_PER_BLOCK = 2048;    // 256 threads x 8 values

static __global__ __launch_bounds__(256) void argmax_blocks_kernel(const uint16_t* __restrict__ x, unsigned n, float* __restrict__ cand_v, unsigned* __restrict__ cand_i)
{
    __shared__ float best_v[4];
    __shared__ unsigned best_i[4];
    float bv = -INFINITY;
    unsigned bi = 0xFFFFFFFFu;
    const unsigned base = blockIdx.x * ARGMAX_PER_BLOCK;
#pragma unroll
    for (int j = 0; j < 8; j++)
    {
        const unsigned i = base + j * 256 + threadIdx.x;
        if (i < n)
        {
            const float v = bf16_bits_to_f32(x[i]);
            if (better(v, i, bv, bi)) { bv = v; bi = i; }
        }
    }
    block_argmax<256>(bv, bi, best_v, best_i);
    if (threadIdx.x == 0) { cand_v[blockIdx.x] = bv; cand_i[blockIdx.x] = bi; }
}

// Picks among the block candidates into *d_index; also advances *d_pos when given.
static __global__ __launch_bounds__(256) void argmax_pick_kernel(const float* __restrict__ cand_v, const unsigned* __restrict__ cand_i, unsigned n_cand,
                                                         int* __restrict__ d_index, int* __restrict__ d_pos)
{
    __shared__ float best_v[4];
    __shared__ unsigned best_i[4];
    float bv = -INFINITY;
    unsigned bi = 0xFFFFFFFFu;
    for (unsigned c = threadIdx.x; c < n_cand; c += 256)
    {
        if (better(cand_v[c], cand_i[c], bv, bi)) { bv = cand_v[c]; bi = cand_i[c]; }
    }
    block_argmax<256>(bv, bi, best_v, best_i);
    if (threadIdx.x == 0)
    {
        *d_index = (int)(bi == 0xFFFFFFFFu ? 0u : bi);
        if (d_pos) { *d_pos += 1; }
    }
}

// The greedy pick from the candidate list a linear launch left behind, the step counter, and the embedding row of
// the picked token for the next step -- one launch.  The first workgroup writes the token and advances *d_pos; every
// workgroup works the pick out for itself (the list is a few KiB) and copies its share of the embedding row.
static __global__ __launch_bounds__(256) void argmax_pick_embed_kernel(const void* __restrict__ workspace, unsigned n, int* __restrict__ d_index, int* __restrict__ d_pos,
                                                               const uint16_t* __restrict__ W, uint16_t* __restrict__ y, int D, int n_rows)
{
    __shared__ float best_v[4];
    __shared__ unsigned best_i[4];
    __shared__ unsigned picked;
    const ArgmaxCandidates c = argmax_candidates((void*)workspace, n);
    const unsigned n_cand = min(*c.count, n / 2u + 16u);
    float bv = -INFINITY;
    unsigned bi = 0xFFFFFFFFu;
    for (unsigned k = threadIdx.x; k < n_cand; k += 256)
    {
        if (better(c.value[k], c.index[k], bv, bi)) { bv = c.value[k]; bi = c.index[k]; }
    }
    block_argmax<256>(bv, bi, best_v, best_i);
    if (threadIdx.x == 0)
    {
        picked = bi == 0xFFFFFFFFu ? 0u : bi;
        if (blockIdx.x == 0)
        {
            *d_index = (int)picked;
            if (d_pos) { *d_pos += 1; }
        }
    }
    __syncthreads();
    if (!W) { return; }
    const int id = min((int)picked, n_rows - 1);
    for (int ch = blockIdx.x * 256 + threadIdx.x; ch * 8 < D; ch += gridDim.x * 256)
    {
        *(u32x4*)(y + ch * 8) = *(const u32x4*)(W + (size_t)id * D + ch * 8);
    }
}

}    // namespace ccq
