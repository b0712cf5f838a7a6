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
// reference's rounding points.  Grid (ceil(T / 32), kv heads); a workgroup of four waves owns 32 tokens (two 16-token
// tiles), wave w the query head kvh * G + w (waves >= G only help with the staging).  Keys and values go through LDS in
// blocks of 64 rows, fetched once per workgroup and pass and shared by the G heads and both token tiles (fetched by every
// wave for itself they cost four times the cache traffic, which bounded the kernel).  Two passes over the keys
// 0 .. pos0 + (last token of the workgroup):
//   pass 1  scores of 16 keys x 16 tokens per v_mfma_f32_16x16x32_bf16 x 4 (key rows as the row operand, the rotated
//           queries as columns: D lane (token = lane % 16, g = lane / 16) holds keys 4 g .. 4 g + 3), rounded to BF16,
//           masked, running (max, sum) per lane, merged over the four lane groups at the end;
//   pass 2  the same scores again, p = bf16(exp(s - max) / sum) -- the probabilities of the whole row, as the reference
//           rounds them -- and y += P V on the matrix cores: the eight probabilities a lane holds for its token (keys
//           4 g .. + 3 and 16 + 4 g .. + 3 of a 32-key slab) are its row operand as they are, because a contraction does not
//           care in which order k is visited when both operands agree; the value operand (column = dim, the same keys)
//           comes from a transposed copy of the value block, two keys per dword.
// Value rows past the last position written so far may hold anything: they are zeroed while staging (0 * NaN is NaN).
constexpr int PF_KEYS = 64;                 // keys per staged block
constexpr int PF_PITCH = 68;                // elements per transposed value row: 64 keys + 4 (34 dwords: 8-byte reads of 16 rows hit 32 distinct banks)
constexpr int PF_KPITCH = 136;              // elements per staged key row: 128 dims + 8 (68 dwords: 16 rows x 16 bytes hit 64 distinct banks)
constexpr int PF_TT = 1;                    // 16-token tiles per workgroup

// expf through the hardware's 2^x (x * log2 e is rounded once more in front of it: a few FP32 ulps, against the BF16
// rounding that follows every use here)
__device__ __forceinline__ float pf_exp(float x) { return __expf(x); }

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every global load in flight (its
// release fence drains the vector-memory counter on this target), which would cancel the two-blocks-ahead prefetch below:
// the kernel then pays a trip to memory per block (1.3 us per 64 keys and pass, whatever the arithmetic costs).
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <int G>
__global__ __launch_bounds__(256) void attn_prefill_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ k_cache, const uint16_t* __restrict__ v_cache,
                                                          uint16_t* __restrict__ y, int n_q, int t_kv, int n_tokens, int pos0, float scale)
{
    __shared__ __attribute__((aligned(16))) uint16_t ks[PF_KEYS * PF_KPITCH];   // [key][dim] of the current block
    __shared__ __attribute__((aligned(16))) uint16_t vt[128 * PF_PITCH];        // [dim][key] of the current block
    const int kvh = blockIdx.y;
    const int t0 = ((int)gridDim.x - 1 - (int)blockIdx.x) * (16 * PF_TT);       // the workgroups that see the most keys go first
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane & 15, g = lane >> 4;
    const int last_token = min(t0 + 16 * PF_TT - 1, n_tokens - 1);
    const int n_keys = pos0 + last_token + 1;                   // keys this workgroup can see
    const int n_written = pos0 + n_tokens;                      // cache rows holding data
    const int n_blocks = (n_keys + PF_KEYS - 1) / PF_KEYS;
    const bool active = wave < G;
    const uint16_t* kbase = k_cache + (size_t)kvh * t_kv * 128;
    const uint16_t* vbase = v_cache + (size_t)kvh * t_kv * 128;

    // the query operands: token tile tt, token j's head, dims 32 c + 8 g .. + 7
    u32x4 qf[PF_TT][4];
    int my_pos[PF_TT];
#pragma unroll
    for (int tt = 0; tt < PF_TT; tt++)
    {
        const int t = min(t0 + tt * 16 + j, n_tokens - 1);
        my_pos[tt] = pos0 + t;
        if (active)
        {
            const uint16_t* qrow = q + ((size_t)t * n_q + kvh * G + wave) * 128 + g * 8;
#pragma unroll
            for (int c = 0; c < 4; c++) { qf[tt][c] = *(const u32x4*)(qrow + c * 32); }
        }
    }
    // staging: thread -> rows and 16-byte pieces of a 64-row block (item = thread + 256 i: key pair 2 p, 2 p + 1 with
    // p = item % 32, dims 8 c .. + 7 with c = item / 32); raw[2 i], raw[2 i + 1] are the two rows' pieces
    auto load_rows = [&](const uint16_t* base, int b, int limit, u32x4 (&raw)[4]) {
#pragma unroll
        for (int i = 0; i < 2; i++)
        {
            const int item = threadIdx.x + i * 256;
            const int row = b * PF_KEYS + 2 * (item & 31);
            // no predicate on the loads (rows past the limit re-read its last row and are zeroed when stored), so that
            // the number of requests in flight is known at every wait
            raw[2 * i] = *(const u32x4*)(base + (size_t)min(row, limit - 1) * 128 + (item >> 5) * 8);
            raw[2 * i + 1] = *(const u32x4*)(base + (size_t)min(row + 1, limit - 1) * 128 + (item >> 5) * 8);
        }
    };
    const u32x4 zero4 = { 0u, 0u, 0u, 0u };
    auto store_keys = [&](int b, int limit, const u32x4 (&raw)[4]) {
#pragma unroll
        for (int i = 0; i < 2; i++)
        {
            const int item = threadIdx.x + i * 256;
            const int row = b * PF_KEYS + 2 * (item & 31);
            uint16_t* dst = ks + 2 * (item & 31) * PF_KPITCH + (item >> 5) * 8;
            *(u32x4*)dst = row < limit ? raw[2 * i] : zero4;
            *(u32x4*)(dst + PF_KPITCH) = row + 1 < limit ? raw[2 * i + 1] : zero4;
        }
    };
    // transposed store, two keys per dword: dim 8 c + e gets (key 2 p, key 2 p + 1) at dword p of its row
    auto store_values = [&](int b, int limit, const u32x4 (&raw)[4]) {
#pragma unroll
        for (int i = 0; i < 2; i++)
        {
            const int item = threadIdx.x + i * 256;
            const int row = b * PF_KEYS + 2 * (item & 31);
            uint32_t* dst = (uint32_t*)vt + (item >> 5) * 8 * (PF_PITCH / 2) + (item & 31);
            const u32x4 lo = row < limit ? raw[2 * i] : zero4, hi = row + 1 < limit ? raw[2 * i + 1] : zero4;
#pragma unroll
            for (int d = 0; d < 4; d++)
            {
                dst[(2 * d) * (PF_PITCH / 2)] = (lo[d] & 0xFFFFu) | (hi[d] << 16);
                dst[(2 * d + 1) * (PF_PITCH / 2)] = (lo[d] >> 16) | (hi[d] & 0xFFFF0000u);
            }
        }
    };
    // scores of the block's four key tiles (16 keys each) against the token tiles: for tile kt the lane gets keys
    // kt * 16 + 4 g + v, v = 0..3, of token j.  All sixteen key operands are read first and the products run over the
    // tiles inside each 32-dim step, so that consecutive matrix-core instructions never wait for each other's sums.
    auto score_block = [&](int b, bool masked, float (&s)[PF_KEYS / 16][PF_TT][4]) {
        u32x4 kf[PF_KEYS / 16][4];
#pragma unroll
        for (int kt = 0; kt < PF_KEYS / 16; kt++)
        {
            const uint16_t* krow = ks + (kt * 16 + j) * PF_KPITCH + g * 8;
#pragma unroll
            for (int c = 0; c < 4; c++) { kf[kt][c] = *(const u32x4*)(krow + c * 32); }
        }
        f32x4 acc[PF_KEYS / 16][PF_TT];
#pragma unroll
        for (int kt = 0; kt < PF_KEYS / 16; kt++)
#pragma unroll
            for (int tt = 0; tt < PF_TT; tt++) { acc[kt][tt] = f32x4{ 0.0f, 0.0f, 0.0f, 0.0f }; }
#pragma unroll
        for (int c = 0; c < 4; c++)
#pragma unroll
            for (int kt = 0; kt < PF_KEYS / 16; kt++)
#pragma unroll
                for (int tt = 0; tt < PF_TT; tt++)
                {
                    acc[kt][tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kf[kt][c]), __builtin_bit_cast(bf16x8, qf[tt][c]), acc[kt][tt], 0, 0, 0);
                }
#pragma unroll
        for (int kt = 0; kt < PF_KEYS / 16; kt++)
#pragma unroll
            for (int tt = 0; tt < PF_TT; tt++)
            {
                // rounded to BF16 by the hardware conversion (round to nearest even, as the integer trick rounds finite values)
                const f32x4 a = acc[kt][tt];
                const bf16x2 r01 = { (__bf16)(scale * a[0]), (__bf16)(scale * a[1]) }, r23 = { (__bf16)(scale * a[2]), (__bf16)(scale * a[3]) };
                const uint32_t w01 = __builtin_bit_cast(uint32_t, r01), w23 = __builtin_bit_cast(uint32_t, r23);
                s[kt][tt][0] = __builtin_bit_cast(float, w01 << 16);
                s[kt][tt][1] = __builtin_bit_cast(float, w01 & 0xFFFF0000u);
                s[kt][tt][2] = __builtin_bit_cast(float, w23 << 16);
                s[kt][tt][3] = __builtin_bit_cast(float, w23 & 0xFFFF0000u);
                if (masked)                                     // only blocks that reach past the workgroup's first token need the test
                {
#pragma unroll
                    for (int v = 0; v < 4; v++)
                    {
                        const int key = b * PF_KEYS + kt * 16 + 4 * g + v;
                        if (key > my_pos[tt]) { s[kt][tt][v] = -INFINITY; }
                    }
                }
            }
    };

    // ---- pass 1: row maximum and sum of exp(s - max)
    float m[PF_TT], l[PF_TT];
#pragma unroll
    for (int tt = 0; tt < PF_TT; tt++) { m[tt] = -INFINITY; l[tt] = 0.0f; }
    // rows are requested two blocks ahead of their use (two register sets, alternating): one block of work does not cover
    // the trip to memory
    u32x4 kraw[2][4], vraw[2][4];
    load_rows(kbase, 0, n_written, kraw[0]);
    load_rows(kbase, min(1, n_blocks - 1), n_written, kraw[1]);
    auto pass1_block = [&](int b, u32x4 (&kr)[4]) {
        lds_barrier();                                        // the previous block's reads are done
        store_keys(b, n_written, kr);
        load_rows(kbase, min(b + 2, n_blocks - 1), n_written, kr);      // unconditional (clamped): the wait counts stay exact
        lds_barrier();
        if (!active) { return; }
        const bool masked = b * PF_KEYS + PF_KEYS - 1 > pos0 + t0;      // some key of the block lies past the first token's position
        // all four key tiles of the block at once: sixteen independent scores per lane and token tile keep the matrix cores
        // and the VALU busy where one tile at a time is a single chain of dependent instructions
        float s[PF_KEYS / 16][PF_TT][4];
        score_block(b, masked, s);
#pragma unroll
        for (int tt = 0; tt < PF_TT; tt++)
        {
            float bm = -INFINITY;
#pragma unroll
            for (int kt = 0; kt < PF_KEYS / 16; kt++)
#pragma unroll
                for (int v = 0; v < 4; v++) { bm = fmaxf(bm, s[kt][tt][v]); }
            if (bm > m[tt])
            {
                l[tt] *= pf_exp(m[tt] - bm);                    // m = -inf: l is 0 and stays 0
                m[tt] = bm;
            }
            if (m[tt] > -INFINITY)
            {
                float sum = 0.0f;
#pragma unroll
                for (int kt = 0; kt < PF_KEYS / 16; kt++)
#pragma unroll
                    for (int v = 0; v < 4; v++) { sum += pf_exp(s[kt][tt][v] - m[tt]); }
                l[tt] += sum;
            }
        }
    };
    for (int b = 0; b < n_blocks; b += 2)
    {
        pass1_block(b, kraw[0]);
        if (b + 1 < n_blocks) { pass1_block(b + 1, kraw[1]); }
    }
    float inv[PF_TT];
#pragma unroll
    for (int tt = 0; tt < PF_TT; tt++)
    {
        // merge the four lane groups of a token (lanes j, j + 16, j + 32, j + 48)
#pragma unroll
        for (int off = 16; off < 64; off <<= 1)
        {
            const float om = __shfl_xor(m[tt], off), ol = __shfl_xor(l[tt], off);
            const float nm = fmaxf(m[tt], om);
            if (nm > -INFINITY) { l[tt] = l[tt] * pf_exp(m[tt] - nm) + ol * pf_exp(om - nm); }
            m[tt] = nm;
        }
        inv[tt] = l[tt] > 0.0f ? 1.0f / l[tt] : 0.0f;
    }

    // ---- pass 2: probabilities and P V
    f32x4 out[PF_TT][8];
#pragma unroll
    for (int tt = 0; tt < PF_TT; tt++)
#pragma unroll
        for (int d = 0; d < 8; d++) { out[tt][d] = f32x4{ 0.0f, 0.0f, 0.0f, 0.0f }; }
    load_rows(kbase, 0, n_written, kraw[0]);
    load_rows(vbase, 0, n_written, vraw[0]);
    load_rows(kbase, min(1, n_blocks - 1), n_written, kraw[1]);
    load_rows(vbase, min(1, n_blocks - 1), n_written, vraw[1]);
    auto pass2_block = [&](int b, u32x4 (&kr)[4], u32x4 (&vr)[4]) {
        lds_barrier();
        store_keys(b, n_written, kr);
        store_values(b, n_written, vr);
        load_rows(kbase, min(b + 2, n_blocks - 1), n_written, kr);
        load_rows(vbase, min(b + 2, n_blocks - 1), n_written, vr);
        lds_barrier();
        if (!active) { return; }
        const bool masked = b * PF_KEYS + PF_KEYS - 1 > pos0 + t0;
        float s[PF_KEYS / 16][PF_TT][4];
        score_block(b, masked, s);
        // exp(-inf) is 0: a masked key gets probability 0 without a test; the pairs are rounded and packed by one conversion each
        bf16x8 pa[PF_KEYS / 32][PF_TT];
#pragma unroll
        for (int slab = 0; slab < PF_KEYS / 32; slab++)
#pragma unroll
            for (int tt = 0; tt < PF_TT; tt++)
            {
                uint32_t pw[4];
#pragma unroll
                for (int h = 0; h < 2; h++)
#pragma unroll
                    for (int v = 0; v < 2; v++)
                    {
                        const float* sv = s[2 * slab + h][tt];
                        const bf16x2 pp = { (__bf16)(pf_exp(sv[2 * v] - m[tt]) * inv[tt]), (__bf16)(pf_exp(sv[2 * v + 1] - m[tt]) * inv[tt]) };
                        pw[2 * h + v] = __builtin_bit_cast(uint32_t, pp);
                    }
                const u32x4 pvec = { pw[0], pw[1], pw[2], pw[3] };      // keys 4 g .. + 3, then 16 + 4 g .. + 3 of the slab
                pa[slab][tt] = __builtin_bit_cast(bf16x8, pvec);
            }
#pragma unroll
        for (int slab = 0; slab < PF_KEYS / 32; slab++)
#pragma unroll
            for (int d = 0; d < 8; d++)
            {
                // value operand: dim 16 d + j, the same eight keys
                const uint16_t* vrow = vt + (16 * d + j) * PF_PITCH + slab * 32 + 4 * g;
                const uint2 va = *(const uint2*)vrow, vb = *(const uint2*)(vrow + 16);
                const u32x4 vvec = { va.x, va.y, vb.x, vb.y };
#pragma unroll
                for (int tt = 0; tt < PF_TT; tt++)
                {
                    out[tt][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa[slab][tt], __builtin_bit_cast(bf16x8, vvec), out[tt][d], 0, 0, 0);
                }
            }
    };
    for (int b = 0; b < n_blocks; b += 2)
    {
        pass2_block(b, kraw[0], vraw[0]);
        if (b + 1 < n_blocks) { pass2_block(b + 1, kraw[1], vraw[1]); }
    }
    if (!active) { return; }
    // D of the last product: lane (dim = 16 d + j, g) holds tokens 4 g .. 4 g + 3 of its tile
#pragma unroll
    for (int tt = 0; tt < PF_TT; tt++)
#pragma unroll
        for (int d = 0; d < 8; d++)
        {
#pragma unroll
            for (int v = 0; v < 4; v++)
            {
                const int t = t0 + tt * 16 + 4 * g + v;
                if (t < n_tokens) { y[((size_t)t * n_q + kvh * G + wave) * 128 + 16 * d + j] = (uint16_t)f32_to_bf16_bits(out[tt][d][v]); }
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
