// Neighbours of the quantized linear for a whole prompt (T tokens at positions pos0 .. pos0 + T - 1, batch 1): what the
// reference's graph runs between the GEMMs when cccc-llm feeds it T tokens at once (scripts/convert_weights.py:488-692,
// cccc-llm/cccc-llm.cpp:589-618), with the same rounding points as the one-token kernels in decode_kernels.h:
//   q/k RMSNorm per head, RoPE at row pos0 + t, cache append          cccc-hip/hip_functions.cpp:1506-1535, :1719-1738
//   attention  scores = bf16(scale * K^T q), keys k > pos0 + t masked, softmax in FP32 over the row -> BF16
//              probabilities, y = bf16(V p)                            cccc/MatrixEx.cpp:3018-3104, hip_functions.cpp:776-804
//   residual   bf16(a + b); SwiGLU  bf16(bf16(g * bf16(sigmoid g)) * u)   hip_functions.cpp:895-908, :722-732, :953-966
// Activations are token-major: row t of a [T][features] BF16 matrix, which is what hip_quant_gemm writes (column-major
// [features x tokens], ldc = features).  gfx950, wave64.
#pragma once
#include "decode_kernels.h"

namespace ccq
{

// ------------------------------------------------------------------------------------------
// Per-head q/k RMSNorm + RoPE + cache append for T tokens.  Grid (n_q + 2 n_kv, T), one wave per (head, token).
//   q [T][n_q][128] -> q_out [T][n_q][128];  k [T][n_kv][128] -> k_cache[h][pos0 + t];  v -> v_cache[h][pos0 + t]
// q_norm_w == nullptr: no per-head norm (both or neither).
static __global__ __launch_bounds__(64) void qk_norm_rope_kv_rows_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ k, const uint16_t* __restrict__ v,
                                                                 const uint16_t* __restrict__ q_norm_w, const uint16_t* __restrict__ k_norm_w,
                                                                 const uint16_t* __restrict__ cos_tab, const uint16_t* __restrict__ sin_tab,
                                                                 uint16_t* __restrict__ q_out, uint16_t* __restrict__ k_cache, uint16_t* __restrict__ v_cache,
                                                                 int n_q, int n_kv, int t_kv, int pos0, float eps)
{
    const int head = blockIdx.x, t = blockIdx.y;
    const int lane = threadIdx.x;
    const int pos = pos0 + t;
    if (head >= n_q + n_kv)
    {
        const int h = head - n_q - n_kv;
        const uint16_t* src = v + ((size_t)t * n_kv + h) * 128;
        uint16_t* dst = v_cache + ((size_t)h * t_kv + pos) * 128;
        dst[lane] = src[lane];
        dst[lane + 64] = src[lane + 64];
        return;
    }
    const bool is_q = head < n_q;
    const int h = is_q ? head : head - n_q;
    const uint16_t* src = is_q ? q + ((size_t)t * n_q + h) * 128 : k + ((size_t)t * n_kv + h) * 128;
    const uint16_t* nw = is_q ? q_norm_w : k_norm_w;
    float l, r;
    norm_rope_head(src, nw, cos_tab + (size_t)pos * 64, sin_tab + (size_t)pos * 64, eps, lane, l, r);
    uint16_t* dst = is_q ? q_out + ((size_t)t * n_q + h) * 128 : k_cache + ((size_t)h * t_kv + pos) * 128;
    dst[lane] = (uint16_t)f32_to_bf16_bits(l);
    dst[lane + 64] = (uint16_t)f32_to_bf16_bits(r);
}

// ------------------------------------------------------------------------------------------
// Causal GQA attention of T query tokens over cache rows 0 .. pos0 + t, head_dim 128, on the matrix cores, with the
// reference's rounding points.  Grid (ceil(T / 16), kv heads); a workgroup of four waves owns 16 tokens, wave w the
// query head kvh * G + w (waves >= G only help to stage V).  Two passes over the keys 0 .. pos0 + (last token of the
// tile):
//   pass 1  scores of 16 keys x 16 tokens per v_mfma_f32_16x16x32_bf16 x 4 (key rows straight from the cache as the row
//           operand, the rotated queries as columns: D lane (token = lane % 16, g = lane / 16) holds keys 4 g .. 4 g + 3),
//           rounded to BF16, masked, running (max, sum) per lane, merged over the four lane groups at the end;
//   pass 2  the same scores again, p = bf16(expf(s - max) / sum) -- the probabilities of the whole row, as the reference
//           rounds them -- and y += P V on the matrix cores: the eight probabilities a lane holds for its token (keys
//           4 g .. + 3 and 16 + 4 g .. + 3 of a 32-key slab) are its row operand as they are, because a contraction does not
//           care in which order k is visited when both operands agree; the value operand (column = dim, the same keys)
//           comes from a transposed copy of the 64-key value block in LDS, shared by the G heads.
// Value rows past the last position written so far may hold anything: they are zeroed while staging (0 * NaN is NaN).
constexpr int PF_KEYS = 64;                 // keys per staged value block
constexpr int PF_PITCH = 66;                // elements per transposed row: 64 keys + 2 (33 dwords, spreads the rows over the banks)

template <int G>
__global__ __launch_bounds__(256) void attn_prefill_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ k_cache, const uint16_t* __restrict__ v_cache,
                                                          uint16_t* __restrict__ y, int n_q, int t_kv, int n_tokens, int pos0, float scale)
{
    __shared__ __attribute__((aligned(16))) uint16_t vt[128 * PF_PITCH];        // [dim][key] of the current block
    const int kvh = blockIdx.y;
    const int t0 = blockIdx.x * 16;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane & 15, g = lane >> 4;
    const int last_token = min(t0 + 15, n_tokens - 1);
    const int n_keys = pos0 + last_token + 1;                   // keys this tile can see
    const int n_written = pos0 + n_tokens;                      // cache rows holding data
    const int my_pos = pos0 + min(t0 + j, n_tokens - 1);        // position of this lane's token
    const bool active = wave < G;
    const uint16_t* kbase = k_cache + (size_t)kvh * t_kv * 128;
    const uint16_t* vbase = v_cache + (size_t)kvh * t_kv * 128;

    // the query operand: token j's head, dims 32 c + 8 g .. + 7
    u32x4 qf[4];
    if (active)
    {
        const uint16_t* qrow = q + ((size_t)min(t0 + j, n_tokens - 1) * n_q + kvh * G + wave) * 128 + g * 8;
#pragma unroll
        for (int c = 0; c < 4; c++) { qf[c] = *(const u32x4*)(qrow + c * 32); }
    }
    // scores of key tile kt (16 keys) against the 16 tokens: lane gets keys kt * 16 + 4 g + v, v = 0..3, of token j
    auto score_tile = [&](int kt, float (&s)[4]) {
        const int row = min(kt * 16 + j, t_kv - 1);
        const uint16_t* krow = kbase + (size_t)row * 128 + g * 8;
        f32x4 acc = { 0.0f, 0.0f, 0.0f, 0.0f };
#pragma unroll
        for (int c = 0; c < 4; c++)
        {
            const u32x4 kf = *(const u32x4*)(krow + c * 32);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kf), __builtin_bit_cast(bf16x8, qf[c]), acc, 0, 0, 0);
        }
#pragma unroll
        for (int v = 0; v < 4; v++)
        {
            const int key = kt * 16 + 4 * g + v;
            s[v] = key <= my_pos ? bf16_round(scale * acc[v]) : -INFINITY;
        }
    };

    // ---- pass 1: row maximum and sum of expf(s - max)
    float m = -INFINITY, l = 0.0f;
    if (active)
    {
        const int n_kt = (n_keys + 15) / 16;
        for (int kt = 0; kt < n_kt; kt++)
        {
            float s[4];
            score_tile(kt, s);
            const float tm = fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3]));
            if (tm > m)
            {
                l *= expf(m - tm);                              // m = -inf: l is 0 and stays 0
                m = tm;
            }
            if (m > -INFINITY)
            {
#pragma unroll
                for (int v = 0; v < 4; v++) { l += expf(s[v] - m); }
            }
        }
        // merge the four lane groups of a token (lanes j, j + 16, j + 32, j + 48)
#pragma unroll
        for (int off = 16; off < 64; off <<= 1)
        {
            const float om = __shfl_xor(m, off), ol = __shfl_xor(l, off);
            const float nm = fmaxf(m, om);
            if (nm > -INFINITY) { l = l * expf(m - nm) + ol * expf(om - nm); }
            m = nm;
        }
    }
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;

    // ---- pass 2: probabilities and P V
    f32x4 out[8];
#pragma unroll
    for (int d = 0; d < 8; d++) { out[d] = f32x4{ 0.0f, 0.0f, 0.0f, 0.0f }; }
    const int n_blocks = (n_keys + PF_KEYS - 1) / PF_KEYS;
    for (int b = 0; b < n_blocks; b++)
    {
        __syncthreads();                                        // the previous block's value reads are done
        // stage V^T: thread -> (key = idx / 16, dims 8 (idx % 16) .. + 7), four keys per thread
#pragma unroll
        for (int i = 0; i < 4; i++)
        {
            const int idx = threadIdx.x + i * 256;
            const int key = idx >> 4, dim0 = (idx & 15) * 8;
            const int row = b * PF_KEYS + key;
            u32x4 raw = { 0u, 0u, 0u, 0u };
            if (row < n_written && row < t_kv) { raw = *(const u32x4*)(vbase + (size_t)row * 128 + dim0); }
#pragma unroll
            for (int d = 0; d < 4; d++)
            {
                vt[(dim0 + 2 * d) * PF_PITCH + key] = (uint16_t)(raw[d] & 0xFFFFu);
                vt[(dim0 + 2 * d + 1) * PF_PITCH + key] = (uint16_t)(raw[d] >> 16);
            }
        }
        __syncthreads();
        if (!active) { continue; }
#pragma unroll
        for (int slab = 0; slab < PF_KEYS / 32; slab++)
        {
            const int key0 = b * PF_KEYS + slab * 32;
            if (key0 >= n_keys) { break; }
            float s0[4], s1[4];
            score_tile(key0 / 16, s0);
            score_tile(key0 / 16 + 1, s1);
            uint32_t pw[4];
#pragma unroll
            for (int v = 0; v < 2; v++)
            {
                const float a0 = s0[2 * v] > -INFINITY ? bf16_round(expf(s0[2 * v] - m) * inv) : 0.0f;
                const float a1 = s0[2 * v + 1] > -INFINITY ? bf16_round(expf(s0[2 * v + 1] - m) * inv) : 0.0f;
                const float b0 = s1[2 * v] > -INFINITY ? bf16_round(expf(s1[2 * v] - m) * inv) : 0.0f;
                const float b1 = s1[2 * v + 1] > -INFINITY ? bf16_round(expf(s1[2 * v + 1] - m) * inv) : 0.0f;
                pw[v] = (__builtin_bit_cast(uint32_t, a0) >> 16) | (__builtin_bit_cast(uint32_t, a1) & 0xFFFF0000u);
                pw[2 + v] = (__builtin_bit_cast(uint32_t, b0) >> 16) | (__builtin_bit_cast(uint32_t, b1) & 0xFFFF0000u);
            }
            const u32x4 pvec = { pw[0], pw[1], pw[2], pw[3] };  // keys 4 g .. + 3, then 16 + 4 g .. + 3 of the slab
            const bf16x8 pa = __builtin_bit_cast(bf16x8, pvec);
#pragma unroll
            for (int d = 0; d < 8; d++)
            {
                // value operand: dim 16 d + j, the same eight keys
                const uint16_t* vrow = vt + (16 * d + j) * PF_PITCH + slab * 32 + 4 * g;
                const uint32_t v0 = *(const uint32_t*)vrow, v1 = *(const uint32_t*)(vrow + 2);
                const uint32_t v2 = *(const uint32_t*)(vrow + 16), v3 = *(const uint32_t*)(vrow + 18);
                const u32x4 vvec = { v0, v1, v2, v3 };
                out[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa, __builtin_bit_cast(bf16x8, vvec), out[d], 0, 0, 0);
            }
        }
    }
    if (!active) { return; }
    // D of the last product: lane (dim = 16 d + j, g) holds tokens 4 g .. 4 g + 3
#pragma unroll
    for (int d = 0; d < 8; d++)
    {
#pragma unroll
        for (int v = 0; v < 4; v++)
        {
            const int t = t0 + 4 * g + v;
            if (t < n_tokens) { y[((size_t)t * n_q + kvh * G + wave) * 128 + 16 * d + j] = (uint16_t)f32_to_bf16_bits(out[d][v]); }
        }
    }
}

// ------------------------------------------------------------------------------------------
// y = bf16(a + b) and the SwiGLU product of the reference's three roundings, eight elements per thread (n % 8 == 0).
static __global__ __launch_bounds__(256) void add_rows_kernel(const u32x4* __restrict__ a, const u32x4* __restrict__ b, u32x4* __restrict__ y, long long n_chunks)
{
    for (long long c = (long long)blockIdx.x * 256 + threadIdx.x; c < n_chunks; c += (long long)gridDim.x * 256)
    {
        const u32x4 va = a[c], vb = b[c];
        u32x4 o;
#pragma unroll
        for (int d = 0; d < 4; d++)
        {
            const float lo = bf16_bits_to_f32(va[d] & 0xFFFFu) + bf16_bits_to_f32(vb[d] & 0xFFFFu);
            const float hi = bf16_bits_to_f32(va[d] >> 16) + bf16_bits_to_f32(vb[d] >> 16);
            o[d] = f32_to_bf16_bits(lo) | (f32_to_bf16_bits(hi) << 16);
        }
        y[c] = o;
    }
}

__device__ __forceinline__ float swiglu_one(float gate, float up)
{
    const float sig = bf16_round(1.0f / (1.0f + expf(-gate)));
    return bf16_round(bf16_round(gate * sig) * up);
}

static __global__ __launch_bounds__(256) void swiglu_rows_kernel(const u32x4* __restrict__ gate, const u32x4* __restrict__ up, u32x4* __restrict__ y, long long n_chunks)
{
    for (long long c = (long long)blockIdx.x * 256 + threadIdx.x; c < n_chunks; c += (long long)gridDim.x * 256)
    {
        const u32x4 vg = gate[c], vu = up[c];
        u32x4 o;
#pragma unroll
        for (int d = 0; d < 4; d++)
        {
            const float lo = swiglu_one(bf16_bits_to_f32(vg[d] & 0xFFFFu), bf16_bits_to_f32(vu[d] & 0xFFFFu));
            const float hi = swiglu_one(bf16_bits_to_f32(vg[d] >> 16), bf16_bits_to_f32(vu[d] >> 16));
            o[d] = f32_to_bf16_bits(lo) | (f32_to_bf16_bits(hi) << 16);
        }
        y[c] = o;
    }
}

}    // namespace ccq
