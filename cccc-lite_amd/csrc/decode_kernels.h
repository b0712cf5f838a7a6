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
};

// Stages the activation vector into LDS in the [step][half][lane] layout of the dot2 kernels,
// applying RMSNorm on the way when asked.  `red` holds THREADS / 64 floats.
template <int THREADS>
__device__ __forceinline__ void stage_decode_activation(const FusedLinearArgs& a, u32x4* xs, float* red)
{
    const int n_steps = (a.K + 1023) / 1024;
    const int n_chunks = n_steps * 128;                      // 16-byte chunks incl. zero padding
    float sumsq = 0.0f;
    for (int c = threadIdx.x; c < n_chunks; c += THREADS)
    {
        u32x4 v = { 0u, 0u, 0u, 0u };
        if (c * 8 < a.K) { v = *(const u32x4*)(a.X + c * 8); }
        if (a.norm_w)
        {
#pragma unroll
            for (int d = 0; d < 4; d++)
            {
                const float lo = bf16_bits_to_f32(v[d] & 0xFFFFu), hi = bf16_bits_to_f32(v[d] >> 16);
                sumsq += lo * lo + hi * hi;
            }
        }
        const int step = c >> 7, in_step = c & 127;
        xs[(step * 2 + (in_step & 1)) * 64 + (in_step >> 1)] = v;
    }
    if (a.norm_w)
    {
        const float total = block_sum<THREADS>(sumsq, red);   // includes the barrier that publishes xs
        const float invstd = rsqrtf(total / (float)a.K + a.norm_eps);
        for (int c = threadIdx.x; c < n_chunks; c += THREADS)
        {
            if (c * 8 < a.K)
            {
                const int step = c >> 7, in_step = c & 127;
                const int slot = (step * 2 + (in_step & 1)) * 64 + (in_step >> 1);
                const u32x4 v = xs[slot];
                const u32x4 w = *(const u32x4*)(a.norm_w + c * 8);
                u32x4 out;
#pragma unroll
                for (int d = 0; d < 4; d++)
                {
                    const float lo = bf16_bits_to_f32(v[d] & 0xFFFFu) * invstd * bf16_bits_to_f32(w[d] & 0xFFFFu);
                    const float hi = bf16_bits_to_f32(v[d] >> 16) * invstd * bf16_bits_to_f32(w[d] >> 16);
                    out[d] = f32_to_bf16_bits(lo) | (f32_to_bf16_bits(hi) << 16);
                }
                xs[slot] = out;
            }
        }
    }
    __syncthreads();
}

template <int WT, int U, int WAVES, bool SCALED>
__global__ __launch_bounds__(WAVES * 64) void gemv8_fused_kernel(const FusedLinearArgs a)
{
    extern __shared__ u32x4 xs[];
    __shared__ float red[WAVES];
    stage_decode_activation<WAVES * 64>(a, xs, red);

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n_steps = (a.K + 1023) / 1024;
    // row groups of two: in pair mode (gate row i, up row i); otherwise two consecutive rows of one segment
    const int g0 = a.pair ? a.n_out[0] : (a.n_out[0] + 1) / 2;
    const int g1 = (a.pair || a.n_segments < 2) ? g0 : g0 + (a.n_out[1] + 1) / 2;
    const int n_groups = (a.pair || a.n_segments < 3) ? g1 : g1 + (a.n_out[2] + 1) / 2;

    for (int g = blockIdx.x * WAVES + wave; g < n_groups; g += gridDim.x * WAVES)
    {
        int seg = 0, row0, row1;
        if (a.pair) { row0 = row1 = g; }
        else
        {
            int local = g;
            if (g >= g1) { seg = 2; local = g - g1; }
            else if (g >= g0) { seg = 1; local = g - g0; }
            row0 = local * 2;
            row1 = min(local * 2 + 1, a.n_out[seg] - 1);
        }
        const uint8_t* w0 = a.W[a.pair ? 0 : seg] + (long long)row0 * a.K + lane * 16;
        const uint8_t* w1 = a.W[a.pair ? 1 : seg] + (long long)row1 * a.K + lane * 16;
        const float s0 = a.w_scale[a.pair ? 0 : seg], s1 = a.w_scale[a.pair ? 1 : seg];
        float acc0 = 0.0f, acc1 = 0.0f;
        for (int st0 = 0; st0 < n_steps; st0 += U)
        {
            u32x4 wa[U], wb[U];
#pragma unroll
            for (int u = 0; u < U; u++)
            {
                wa[u] = wb[u] = u32x4{ 0u, 0u, 0u, 0u };
                if ((st0 + u) * 1024 + lane * 16 < a.K)
                {
                    wa[u] = __builtin_nontemporal_load((const u32x4*)(w0 + (st0 + u) * 1024));
                    wb[u] = __builtin_nontemporal_load((const u32x4*)(w1 + (st0 + u) * 1024));
                }
            }
#pragma unroll
            for (int u = 0; u < U; u++)
            {
                if (st0 + u < n_steps)
                {
                    const u32x4 x0 = xs[((st0 + u) * 2 + 0) * 64 + lane];
                    const u32x4 x1 = xs[((st0 + u) * 2 + 1) * 64 + lane];
#pragma unroll
                    for (int d = 0; d < 4; d++)
                    {
                        const u32x4& xv = (d < 2) ? x0 : x1;
                        bf16x2 p01, p23;
                        fp8x4_to_bf16<WT, SCALED>(wa[u][d], s0, p01, p23);
                        acc0 = dot2_bf16(p01, xv[(d & 1) * 2 + 0], acc0);
                        acc0 = dot2_bf16(p23, xv[(d & 1) * 2 + 1], acc0);
                        fp8x4_to_bf16<WT, SCALED>(wb[u][d], s1, p01, p23);
                        acc1 = dot2_bf16(p01, xv[(d & 1) * 2 + 0], acc1);
                        acc1 = dot2_bf16(p23, xv[(d & 1) * 2 + 1], acc1);
                    }
                }
            }
        }
        const float t0 = wave_sum(acc0), t1 = wave_sum(acc1);
        if (lane == 0)
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
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// Standalone neighbours with the reference's signatures (BF16)

static __global__ __launch_bounds__(256) void rms_norm_bf16_kernel(const uint16_t* __restrict__ X, uint16_t* __restrict__ Y, const uint16_t* __restrict__ scale,
                                                           float* __restrict__ invstd_out, unsigned inner, float eps)
{
    __shared__ float red[4];
    const uint16_t* x = X + (size_t)blockIdx.x * inner;
    uint16_t* y = Y + (size_t)blockIdx.x * inner;
    float sumsq = 0.0f;
    for (unsigned i = threadIdx.x; i < inner; i += 256)
    {
        const float v = bf16_bits_to_f32(x[i]);
        sumsq += v * v;
    }
    const float invstd = rsqrtf(block_sum<256>(sumsq, red) / (float)inner + eps);
    if (threadIdx.x == 0 && invstd_out) { invstd_out[blockIdx.x] = invstd; }
    for (unsigned i = threadIdx.x; i < inner; i += 256)
    {
        const float sc = scale ? bf16_bits_to_f32(scale[i]) : 1.0f;
        y[i] = (uint16_t)f32_to_bf16_bits(bf16_bits_to_f32(x[i]) * invstd * sc);
    }
}

static __global__ __launch_bounds__(256) void rope_bf16_kernel(const uint16_t* __restrict__ X, uint16_t* __restrict__ Y, const uint16_t* __restrict__ cos_tab,
                                                       const uint16_t* __restrict__ sin_tab, unsigned D, unsigned T, unsigned B, unsigned pos_offset)
{
    const unsigned half_d = D / 2;
    const unsigned idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= half_d * T * B) { return; }
    const unsigned i = idx % half_d;
    const unsigned bt = idx / half_d;
    const unsigned t = bt % T;
    const size_t base = (size_t)bt * D;
    const size_t tab = (size_t)(t + pos_offset) * half_d + i;
    const float c = bf16_bits_to_f32(cos_tab[tab]), s = bf16_bits_to_f32(sin_tab[tab]);
    const float xl = bf16_bits_to_f32(X[base + i]), xr = bf16_bits_to_f32(X[base + half_d + i]);
    Y[base + i] = (uint16_t)f32_to_bf16_bits(xl * c - xr * s);
    Y[base + half_d + i] = (uint16_t)f32_to_bf16_bits(xr * c + xl * s);
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
    const float invstd = rsqrtf(wave_sum(xl * xl + xr * xr) / 128.0f + eps);
    const float nl = bf16_round(xl * invstd * bf16_bits_to_f32(nw[lane]));
    const float nr = bf16_round(xr * invstd * bf16_bits_to_f32(nw[lane + 64]));
    const float c = bf16_bits_to_f32(cos_tab[(size_t)pos * 64 + lane]), s = bf16_bits_to_f32(sin_tab[(size_t)pos * 64 + lane]);
    uint16_t* dst = is_q ? q_out + h * 128 : k_cache + ((size_t)h * t_kv + pos) * 128;
    dst[lane] = (uint16_t)f32_to_bf16_bits(nl * c - nr * s);
    dst[lane + 64] = (uint16_t)f32_to_bf16_bits(nr * c + nl * s);
}

// ------------------------------------------------------------------------------------------
// GQA decode attention, head_dim 128, group of G = n_q / n_kv query heads per KV head.
// Pass 1: scores[qh][t] = bf16(scale * k_t . q_qh) for t <= pos.  16 lanes share a key (8 dims each),
// a wave covers 4 keys per 1 KiB load; a workgroup covers 64 keys of one KV head.
template <int G>
__global__ __launch_bounds__(256) void attn_scores_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ k_cache, uint16_t* __restrict__ scores,
                                                         int t_kv, const int* __restrict__ d_pos, float scale)
{
    const int kvh = blockIdx.y;
    const int n_keys = min(max(*d_pos, 0), t_kv - 1) + 1;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane & 15;              // which 8 dims
    const int key_in_wave = lane >> 4;
    float qv[G][8];
#pragma unroll
    for (int gq = 0; gq < G; gq++)
    {
        const u32x4 raw = *(const u32x4*)(q + (size_t)(kvh * G + gq) * 128 + sub * 8);
#pragma unroll
        for (int d = 0; d < 4; d++)
        {
            qv[gq][2 * d] = bf16_bits_to_f32(raw[d] & 0xFFFFu);
            qv[gq][2 * d + 1] = bf16_bits_to_f32(raw[d] >> 16);
        }
    }
#pragma unroll
    for (int it = 0; it < 4; it++)
    {
        const int t = blockIdx.x * 64 + wave * 16 + it * 4 + key_in_wave;
        u32x4 raw = { 0u, 0u, 0u, 0u };
        if (t < n_keys) { raw = *(const u32x4*)(k_cache + ((size_t)kvh * t_kv + t) * 128 + sub * 8); }
        float kf[8];
#pragma unroll
        for (int d = 0; d < 4; d++)
        {
            kf[2 * d] = bf16_bits_to_f32(raw[d] & 0xFFFFu);
            kf[2 * d + 1] = bf16_bits_to_f32(raw[d] >> 16);
        }
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
            if (sub == 0 && t < n_keys) { scores[(size_t)(kvh * G + gq) * t_kv + t] = (uint16_t)f32_to_bf16_bits(scale * dot); }
        }
    }
}

// Pass 2: softmax statistics over all scores of each query head (recomputed by every workgroup: the
// row is at most a few KiB), probabilities p_t = bf16(expf(s_t - max) * (1 / sum)), partial outputs
// over this workgroup's slice of timesteps: partial[split][qh][128] (FP32).  A workgroup reads its
// V slice once for all G query heads.
template <int G>
__global__ __launch_bounds__(256) void attn_pv_kernel(const uint16_t* __restrict__ scores, const uint16_t* __restrict__ v_cache, float* __restrict__ partial,
                                                     int t_kv, const int* __restrict__ d_pos, int n_splits, int n_q)
{
    __shared__ float red[4];
    __shared__ float acc_lds[16][G][128];   // [key slot in workgroup][head][dim]
    const int kvh = blockIdx.y, split = blockIdx.x;
    const int n_keys = min(max(*d_pos, 0), t_kv - 1) + 1;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane & 15, key_in_wave = lane >> 4;

    float maxv[G], inv_sum[G];
#pragma unroll
    for (int gq = 0; gq < G; gq++)
    {
        const uint16_t* s = scores + (size_t)(kvh * G + gq) * t_kv;
        float m = -3.0e38f;
        for (int t = threadIdx.x; t < n_keys; t += 256) { m = fmaxf(m, bf16_bits_to_f32(s[t])); }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) { m = fmaxf(m, __shfl_xor(m, off)); }
        if (lane == 0) { red[wave] = m; }
        __syncthreads();
        m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        __syncthreads();
        float sum = 0.0f;
        for (int t = threadIdx.x; t < n_keys; t += 256) { sum += expf(bf16_bits_to_f32(s[t]) - m); }
        sum = block_sum<256>(sum, red);
        maxv[gq] = m;
        inv_sum[gq] = sum > 0.0f ? 1.0f / sum : 0.0f;
    }

    const int per_split = (n_keys + n_splits - 1) / n_splits;
    const int t_lo = split * per_split, t_hi = min(t_lo + per_split, n_keys);
    float acc[G][8];
#pragma unroll
    for (int gq = 0; gq < G; gq++)
#pragma unroll
        for (int d = 0; d < 8; d++) { acc[gq][d] = 0.0f; }
    for (int t = t_lo + wave * 4 + key_in_wave; t < t_hi; t += 16)
    {
        const u32x4 raw = *(const u32x4*)(v_cache + ((size_t)kvh * t_kv + t) * 128 + sub * 8);
        float vf[8];
#pragma unroll
        for (int d = 0; d < 4; d++)
        {
            vf[2 * d] = bf16_bits_to_f32(raw[d] & 0xFFFFu);
            vf[2 * d + 1] = bf16_bits_to_f32(raw[d] >> 16);
        }
#pragma unroll
        for (int gq = 0; gq < G; gq++)
        {
            const float s = bf16_bits_to_f32(scores[(size_t)(kvh * G + gq) * t_kv + t]);
            const float p = bf16_round(expf(s - maxv[gq]) * inv_sum[gq]);
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
        partial[((size_t)split * n_q + kvh * G + gq) * 128 + d] = total;
    }
}

// y[i] = bf16(sum_s partial[s][i])
static __global__ __launch_bounds__(256) void sum_partials_kernel(const float* __restrict__ partial, uint16_t* __restrict__ y, int n_splits, int n)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n) { return; }
    float total = 0.0f;
    for (int s = 0; s < n_splits; s++) { total += partial[(size_t)s * n + i]; }
    y[i] = (uint16_t)f32_to_bf16_bits(total);
}

// Index of the largest BF16 value (lowest index on ties) into *d_index; also advances *d_pos when given.
static __global__ __launch_bounds__(1024) void argmax_bf16_kernel(const uint16_t* __restrict__ x, unsigned n, int* __restrict__ d_index, int* __restrict__ d_pos)
{
    __shared__ float best_v[16];
    __shared__ unsigned best_i[16];
    float bv = -3.4e38f;
    unsigned bi = 0xFFFFFFFFu;
    for (unsigned i = threadIdx.x; i < n; i += 1024)
    {
        const float v = bf16_bits_to_f32(x[i]);
        if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1)
    {
        const float ov = __shfl_xor(bv, off);
        const unsigned oi = __shfl_xor(bi, off);
        if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    if ((threadIdx.x & 63) == 0) { best_v[threadIdx.x >> 6] = bv; best_i[threadIdx.x >> 6] = bi; }
    __syncthreads();
    if (threadIdx.x == 0)
    {
        for (int w = 1; w < 16; w++)
        {
            if (best_v[w] > bv || (best_v[w] == bv && best_i[w] < bi)) { bv = best_v[w]; bi = best_i[w]; }
        }
        *d_index = (int)(bi == 0xFFFFFFFFu ? 0u : bi);
        if (d_pos) { *d_pos += 1; }
    }
}

}    // namespace ccq
