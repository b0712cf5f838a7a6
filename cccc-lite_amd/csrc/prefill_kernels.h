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
// Per-head q/k RMSNorm + RoPE + cache append for T tokens.  Grid (ceil((n_q + 2 n_kv) / 4), T), one wave per (head, token)
// and four of them per workgroup (one wave per workgroup -- 98 k tiny workgroups for 2048 tokens -- ran at a quarter of
// the rate).  The arithmetic per head is the one-token kernel's, lane for lane.
//   q [T][n_q][128] -> q_out [T][n_q][128];  k [T][n_kv][128] -> k_cache[h][pos0 + t];  v -> v_cache[h][pos0 + t]
// q_norm_w == nullptr: no per-head norm (both or neither).
static __global__ __launch_bounds__(256) void qk_norm_rope_kv_rows_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ k, const uint16_t* __restrict__ v,
                                                                  const uint16_t* __restrict__ q_norm_w, const uint16_t* __restrict__ k_norm_w,
                                                                  const uint16_t* __restrict__ cos_tab, const uint16_t* __restrict__ sin_tab,
                                                                  uint16_t* __restrict__ q_out, uint16_t* __restrict__ k_cache, uint16_t* __restrict__ v_cache,
                                                                  int n_q, int n_kv, int t_kv, int pos0, float eps)
{
    const int head = blockIdx.x * 4 + (threadIdx.x >> 6), t = blockIdx.y;
    const int lane = threadIdx.x & 63;
    const int pos = pos0 + t;
    if (head >= n_q + 2 * n_kv) { return; }
    if (head >= n_q + n_kv)
    {
        const int h = head - n_q - n_kv;
        const uint32_t* src = (const uint32_t*)(v + ((size_t)t * n_kv + h) * 128);
        uint32_t* dst = (uint32_t*)(v_cache + ((size_t)h * t_kv + pos) * 128);
        dst[lane] = src[lane];
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
// reference's rounding points.  Grid ceil(T / 16) x kv heads, one-dimensional; a workgroup of four waves owns 16 tokens of the
// G query heads of one kv head: a wave takes two heads (one when G = 1) and one half -- 32 keys -- of every staged block, so
// that a key or value operand read from LDS serves two products and the halves of a head meet once at the end (waves left
// over only help with the staging).  Keys and values go through LDS in blocks of 64 rows,
// fetched once per workgroup and pass and shared by the G heads.  Two passes over the keys 0 .. pos0 + (last token of
// the workgroup):
//   pass 1  scores of 16 keys x 16 tokens per v_mfma_f32_16x16x32_bf16 x 4 (key rows as the row operand, the rotated
//           queries as columns: D lane (token = lane % 16, g = lane / 16) holds keys 4 g .. 4 g + 3), rounded to BF16,
//           masked, running (max, sum) per lane, merged over the four lane groups at the end;
//   pass 2  the same scores again, p = bf16(exp(s - max) / sum) -- the probabilities of the whole row, as the reference
//           rounds them -- and y += P V on the matrix cores: the eight probabilities a lane holds for its token (keys
//           4 g .. + 3 and 16 + 4 g .. + 3 of a 32-key slab) are its row operand as they are, because a contraction does not
//           care in which order k is visited when both operands agree; the value operand (column = dim, the same keys)
//           comes from a transposed copy of the value block, two keys per dword.
// Both passes are software-pipelined over two LDS buffers: while the VALU turns the raw scores of block b into statistics
// or probabilities, the matrix cores already multiply block b + 1, whose keys were staged one iteration earlier; the
// rows of block b + 2 travel from memory meanwhile and are stored behind the iteration's single barrier.
// Value rows past the last position written so far may hold anything: they are zeroed while staging (0 * NaN is NaN).
constexpr int PF_KEYS = 64;                 // keys per staged block
constexpr int PF_PITCH = 68;                // elements per transposed value row: 64 keys + 4 (34 dwords: 8-byte reads of 16 rows hit 32 distinct banks; 72 measured the same)
constexpr int PF_KPITCH = 136;              // elements per staged key row: 128 dims + 8 (68 dwords: 16 rows x 16 bytes hit 64 distinct banks)
constexpr float PF_LOG2E = 1.4426950408889634f;

// 2^x on the hardware unit.  exp(s - m) is taken as 2^(s log2 e - m log2 e) with one fused multiply-add in front: a few FP32
// ulps from expf, against the BF16 rounding that follows every use here.
__device__ __forceinline__ float pf_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Two FP32 values rounded to BF16 (nearest even) into one dword, low half first.  Spelled as the instruction because the
// compiler, seeing the halves used separately afterwards, converts each value with an instruction of its own.  The compiler
// keeps the wait states between a VALU write and a matrix-core read only for instructions it emits itself: a result of
// this block consumed by the very next matrix-core instruction arrived stale in some lanes (NaN rows).  The block
// therefore carries its own wait states behind the conversion, so that the result is safe for whichever instruction
// follows; the callers here hand it to VALU code, and matrix-core operands are still built with (__bf16) casts.
__device__ __forceinline__ uint32_t pf_pack_bf16(float lo, float hi)
{
    uint32_t r;
    asm("v_cvt_pk_bf16_f32 %0, %1, %2\n\ts_nop 1" : "=v"(r) : "v"(lo), "v"(hi));
    return r;
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every global load in flight (its
// release fence drains the vector-memory counter on this target), which would cancel the prefetch below: the kernel
// then pays a trip to memory per block.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <int G>
__global__ __launch_bounds__(256, 2) void attn_prefill_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ k_cache, const uint16_t* __restrict__ v_cache,
                                                             uint16_t* __restrict__ y, int n_q, int t_kv, int n_tokens, int pos0, float scale)
{
    constexpr int H = G >= 2 ? 2 : 1;           // query heads per wave
    constexpr int NW = 2 * (G / H);             // waves that compute: (head group, key half)
    static_assert(G == 1 || G == 2 || G == 4, "query heads per kv head");
    __shared__ __attribute__((aligned(16))) uint16_t ks[2][PF_KEYS * PF_KPITCH];   // [key][dim] of two blocks
    __shared__ __attribute__((aligned(16))) uint16_t vt[2][128 * PF_PITCH];        // [dim][key] of two blocks
    __shared__ float2 stat[4][H][16];                                              // (max, sum) per wave, head and token
    // Consecutive workgroups go to the eight XCDs in turn, each with an L2 of its own: with the kv head as the fastest index
    // an XCD serves few heads (one, with eight of them) and their keys and values stay in its L2 for all token tiles.
    const int n_kv = n_q / G;
    const int kvh = blockIdx.x % n_kv;
    const int t0 = ((int)gridDim.x / n_kv - 1 - (int)blockIdx.x / n_kv) * 16;   // the workgroups that see the most keys go first
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane & 15, g = lane >> 4;
    const int last_token = min(t0 + 15, n_tokens - 1);
    const int n_keys = pos0 + last_token + 1;                   // keys this workgroup can see
    const int n_written = pos0 + n_tokens;                      // cache rows holding data
    const int n_blocks = (n_keys + PF_KEYS - 1) / PF_KEYS;
    const bool active = wave < NW;
    const int hg = wave >> 1, kh = wave & 1;                    // head group; which 32 keys of every block
    const int head0 = kvh * G + hg * H;                         // first of the wave's heads
    const uint16_t* kbase = k_cache + (size_t)kvh * t_kv * 128;
    const uint16_t* vbase = v_cache + (size_t)kvh * t_kv * 128;

    // the query operands: token j, head head0 + h, dims 32 c + 8 g .. + 7
    u32x4 qf[H][4];
    const int my_pos = pos0 + min(t0 + j, n_tokens - 1);
    if (active)
    {
#pragma unroll
        for (int h = 0; h < H; h++)
        {
            const uint16_t* qrow = q + ((size_t)min(t0 + j, n_tokens - 1) * n_q + head0 + h) * 128 + g * 8;
#pragma unroll
            for (int c = 0; c < 4; c++) { qf[h][c] = *(const u32x4*)(qrow + c * 32); }
        }
    }
    // staging: a thread moves two 16-byte pieces (dims 8 c .. + 7 and 64 + 8 c .. + 7, c = thread / 32) of two rows (keys
    // 2 p, 2 p + 1 of the block, p = thread % 32): raw[2 i], raw[2 i + 1] are the two rows' pieces i.  A block index past the
    // last block is clamped to it; rows past the last written one re-read it (no predicate on the loads) and are zeroed
    // when stored.  Addresses are a uniform base plus a 32-bit offset per lane.
    const int p2 = 2 * (threadIdx.x & 31), c8 = (threadIdx.x >> 5) * 8;
    auto load_rows = [&](const uint16_t* base, int b, u32x4 (&raw)[4]) {
        const int row = min(b, n_blocks - 1) * PF_KEYS + p2;
        const uint32_t o0 = (uint32_t)min(row, n_written - 1) * 256u + c8 * 2, o1 = (uint32_t)min(row + 1, n_written - 1) * 256u + c8 * 2;
        const char* base8 = (const char*)base;
        raw[0] = *(const u32x4*)(base8 + o0);
        raw[1] = *(const u32x4*)(base8 + o1);
        raw[2] = *(const u32x4*)(base8 + o0 + 128);
        raw[3] = *(const u32x4*)(base8 + o1 + 128);
    };
    const u32x4 zero4 = { 0u, 0u, 0u, 0u };
    auto store_keys = [&](int buf, int b, const u32x4 (&raw)[4]) {
        const int row = min(b, n_blocks - 1) * PF_KEYS + p2;
        uint16_t* dst = ks[buf] + p2 * PF_KPITCH + c8;
        if (row + PF_KEYS <= n_written)                         // (a sufficient test: no row of the block needs zeroing)
        {
            *(u32x4*)dst = raw[0];
            *(u32x4*)(dst + PF_KPITCH) = raw[1];
            *(u32x4*)(dst + 64) = raw[2];
            *(u32x4*)(dst + PF_KPITCH + 64) = raw[3];
        }
        else
        {
            const bool in0 = row < n_written, in1 = row + 1 < n_written;
            *(u32x4*)dst = in0 ? raw[0] : zero4;
            *(u32x4*)(dst + PF_KPITCH) = in1 ? raw[1] : zero4;
            *(u32x4*)(dst + 64) = in0 ? raw[2] : zero4;
            *(u32x4*)(dst + PF_KPITCH + 64) = in1 ? raw[3] : zero4;
        }
    };
    // transposed store, two keys per dword: dim 8 c + e gets (key 2 p, key 2 p + 1) at dword p of its row
    auto store_values = [&](int buf, int b, const u32x4 (&raw)[4]) {
        const int row = min(b, n_blocks - 1) * PF_KEYS + p2;
        const bool whole = (min(b, n_blocks - 1) + 1) * PF_KEYS <= n_written;       // uniform: no row of the block needs zeroing
        const bool in0 = whole || row < n_written, in1 = whole || row + 1 < n_written;
#pragma unroll
        for (int i = 0; i < 2; i++)
        {
            uint32_t* dst = (uint32_t*)vt[buf] + (c8 + 64 * i) * (PF_PITCH / 2) + (p2 >> 1);
            u32x4 lo = raw[2 * i], hi = raw[2 * i + 1];
            if (!whole)
            {
                lo = in0 ? lo : zero4;
                hi = in1 ? hi : zero4;
            }
#pragma unroll
            for (int d = 0; d < 4; d++)
            {
                dst[(2 * d) * (PF_PITCH / 2)] = __builtin_amdgcn_perm(hi[d], lo[d], 0x05040100u);       // low halves of both keys
                dst[(2 * d + 1) * (PF_PITCH / 2)] = __builtin_amdgcn_perm(hi[d], lo[d], 0x07060302u);   // high halves
            }
        }
    };
    // raw scores of the wave's two key tiles (keys 32 kh + 16 kt + ..) of a staged block against the token tile, for its H
    // heads: for tile kt the lane gets keys 32 kh + 16 kt + 4 g + v, v = 0..3, of token j.  A key operand read from LDS
    // serves H products; all eight are read first and the products run over tiles and heads inside each 32-dim step, so
    // that consecutive matrix-core instructions never wait for each other's sums.
    auto score_products = [&](int buf, f32x4 (&acc)[H][2]) {
        u32x4 kf[2][4];
#pragma unroll
        for (int kt = 0; kt < 2; kt++)
        {
            const uint16_t* krow = ks[buf] + (kh * 32 + kt * 16 + j) * PF_KPITCH + g * 8;
#pragma unroll
            for (int c = 0; c < 4; c++) { kf[kt][c] = *(const u32x4*)(krow + c * 32); }
        }
#pragma unroll
        for (int h = 0; h < H; h++)
#pragma unroll
            for (int kt = 0; kt < 2; kt++) { acc[h][kt] = f32x4{ 0.0f, 0.0f, 0.0f, 0.0f }; }
#pragma unroll
        for (int c = 0; c < 4; c++)
#pragma unroll
            for (int kt = 0; kt < 2; kt++)
#pragma unroll
                for (int h = 0; h < H; h++)
                {
                    acc[h][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kf[kt][c]), __builtin_bit_cast(bf16x8, qf[h][c]), acc[h][kt], 0, 0, 0);
                }
    };
    // scaled, rounded to BF16 by the hardware conversion (round to nearest even, as the integer trick rounds finite
    // values) and masked: only blocks that reach past the workgroup's first token need the test
    auto score_round = [&](const f32x4 (&acc)[H][2], int b, auto masked_c, float (&s)[H][2][4]) {
        constexpr bool masked = decltype(masked_c)::value;
#pragma unroll
        for (int h = 0; h < H; h++)
#pragma unroll
            for (int kt = 0; kt < 2; kt++)
            {
                const f32x4 a = acc[h][kt];
                const uint32_t w01 = pf_pack_bf16(scale * a[0], scale * a[1]), w23 = pf_pack_bf16(scale * a[2], scale * a[3]);
                s[h][kt][0] = __builtin_bit_cast(float, w01 << 16);
                s[h][kt][1] = __builtin_bit_cast(float, w01 & 0xFFFF0000u);
                s[h][kt][2] = __builtin_bit_cast(float, w23 << 16);
                s[h][kt][3] = __builtin_bit_cast(float, w23 & 0xFFFF0000u);
                if (masked)
                {
#pragma unroll
                    for (int v = 0; v < 4; v++)
                    {
                        if (b * PF_KEYS + kh * 32 + kt * 16 + 4 * g + v > my_pos) { s[h][kt][v] = -INFINITY; }
                    }
                }
            }
    };

    // ---- pass 1: row maximum and sum of exp(s - max), per lane over its keys
    float m[H], l[H];
#pragma unroll
    for (int h = 0; h < H; h++) { m[h] = -INFINITY; l[h] = 0.0f; }
    u32x4 kraw[4], vraw[4];
    f32x4 cur[H][2], next[H][2];
    // blocks 0 .. n_plain - 1 end at or before the first token's position and need no mask test (one or two blocks do)
    const int n_plain = min((pos0 + t0 + 1) / PF_KEYS, n_blocks);
    // prologue: block 0 staged and multiplied, block 1 staged, block 2 on its way
    load_rows(kbase, 0, kraw);
    store_keys(0, 0, kraw);
    load_rows(kbase, 1, kraw);
    lds_barrier();
    if (active) { score_products(0, cur); }
    store_keys(1, 1, kraw);
    load_rows(kbase, 2, kraw);
    lds_barrier();
    // iteration b: ks[(b + 1) & 1] holds block b + 1, `cur` the raw scores of block b, kraw block b + 2 in flight
    auto pass1_block = [&](int b, auto masked_c) {
        if (active)
        {
            score_products((b + 1) & 1, next);
            float s[H][2][4];
            score_round(cur, b, masked_c, s);
#pragma unroll
            for (int h = 0; h < H; h++)
            {
                float bm = -INFINITY;
#pragma unroll
                for (int kt = 0; kt < 2; kt++)
#pragma unroll
                    for (int v = 0; v < 4; v++) { bm = fmaxf(bm, s[h][kt][v]); }
                const float nm = fmaxf(m[h], bm);
                // nm = -inf: nothing visible to this lane yet, every term below is 2^(-inf) = 0 with the offset at 0
                const float off = nm > -INFINITY ? -nm * PF_LOG2E : 0.0f;
                l[h] = nm == m[h] ? l[h] : l[h] * pf_exp2(fmaf(m[h], PF_LOG2E, off));
                m[h] = nm;
                float sum = 0.0f;
#pragma unroll
                for (int kt = 0; kt < 2; kt++)
#pragma unroll
                    for (int v = 0; v < 4; v++) { sum += pf_exp2(fmaf(s[h][kt][v], PF_LOG2E, off)); }
                l[h] += sum;
            }
        }
        store_keys(b & 1, b + 2, kraw);                         // block b's buffer: its reads ended before the last barrier
        load_rows(kbase, b + 3, kraw);
        lds_barrier();
#pragma unroll
        for (int h = 0; h < H; h++)
#pragma unroll
            for (int kt = 0; kt < 2; kt++) { cur[h][kt] = next[h][kt]; }
    };
    // two copies of the iteration, with and without the mask test, each one straight run of instructions
    for (int b = 0; b < n_plain; b++) { pass1_block(b, std::false_type{}); }
    for (int b = n_plain; b < n_blocks; b++) { pass1_block(b, std::true_type{}); }
    // merge the four lane groups of a token (lanes j, j + 16, j + 32, j + 48), then the two waves of a head group
    auto merge = [&](float& ma, float& la, float mb, float lb) {
        const float nm = fmaxf(ma, mb);
        if (nm > -INFINITY) { la = la * pf_exp2((ma - nm) * PF_LOG2E) + lb * pf_exp2((mb - nm) * PF_LOG2E); }
        ma = nm;
    };
#pragma unroll
    for (int h = 0; h < H; h++)
    {
#pragma unroll
        for (int off = 16; off < 64; off <<= 1) { merge(m[h], l[h], __shfl_xor(m[h], off), __shfl_xor(l[h], off)); }
        if (active && g == 0) { stat[wave][h][j] = make_float2(m[h], l[h]); }
    }
    lds_barrier();
    float poff[H];
#pragma unroll
    for (int h = 0; h < H; h++)
    {
        if (active)
        {
            const float2 other = stat[wave ^ 1][h][j];
            merge(m[h], l[h], other.x, other.y);
        }
        // p = 2^(s log2 e - (m log2 e + log2 l)): the division by the sum rides in the exponent
        poff[h] = l[h] > 0.0f ? -(m[h] * PF_LOG2E + __builtin_amdgcn_logf(l[h])) : -INFINITY;
    }

    // ---- pass 2: probabilities and P V, per wave over its half of the keys
    f32x4 out[H][8];
#pragma unroll
    for (int h = 0; h < H; h++)
#pragma unroll
        for (int d = 0; d < 8; d++) { out[h][d] = f32x4{ 0.0f, 0.0f, 0.0f, 0.0f }; }
    load_rows(kbase, 0, kraw);
    load_rows(vbase, 0, vraw);
    store_keys(0, 0, kraw);
    load_rows(kbase, 1, kraw);
    lds_barrier();
    if (active) { score_products(0, cur); }
    store_keys(1, 1, kraw);
    store_values(0, 0, vraw);
    load_rows(kbase, 2, kraw);
    load_rows(vbase, 1, vraw);
    lds_barrier();
    // iteration b: ks[(b + 1) & 1] holds key block b + 1, vt[b & 1] value block b; kraw = keys b + 2, vraw = values b + 1 in flight
    auto pass2_block = [&](int b, auto masked_c) {
        if (active)
        {
            score_products((b + 1) & 1, next);
            // value operands (dim 16 d + j, the lane's eight keys 32 kh + 4 g .. + 3 and + 16) are read ahead of their use
            u32x4 vf[8];
#pragma unroll
            for (int d = 0; d < 8; d++)
            {
                const uint16_t* vrow = vt[b & 1] + (16 * d + j) * PF_PITCH + kh * 32 + 4 * g;
                const uint2 va = *(const uint2*)vrow, vb = *(const uint2*)(vrow + 16);
                vf[d] = u32x4{ va.x, va.y, vb.x, vb.y };
            }
            float s[H][2][4];
            score_round(cur, b, masked_c, s);
            // 2^(-inf) is 0: a masked key gets probability 0 without a test; the pairs are rounded and packed by one conversion each
#pragma unroll
            for (int h = 0; h < H; h++)
            {
                uint32_t pw[4];
#pragma unroll
                for (int kt = 0; kt < 2; kt++)
#pragma unroll
                    for (int v = 0; v < 2; v++)
                    {
                        const float* sv = s[h][kt];
                        // (converted by the compiler's own instruction, not pf_pack_bf16: the result feeds a matrix-core instruction, and
                        // only for instructions it knows does the compiler keep the wait states between the two)
                        const bf16x2 pp = { (__bf16)pf_exp2(fmaf(sv[2 * v], PF_LOG2E, poff[h])), (__bf16)pf_exp2(fmaf(sv[2 * v + 1], PF_LOG2E, poff[h])) };
                        pw[2 * kt + v] = __builtin_bit_cast(uint32_t, pp);
                    }
                const u32x4 pvec = { pw[0], pw[1], pw[2], pw[3] };      // keys 4 g .. + 3, then 16 + 4 g .. + 3 of the wave's 32
                const bf16x8 pa = __builtin_bit_cast(bf16x8, pvec);
#pragma unroll
                for (int d = 0; d < 8; d++)
                {
                    out[h][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa, __builtin_bit_cast(bf16x8, vf[d]), out[h][d], 0, 0, 0);
                }
            }
        }
        store_keys(b & 1, b + 2, kraw);
        store_values((b + 1) & 1, b + 1, vraw);                 // held value block b - 1, read before the last barrier
        load_rows(kbase, b + 3, kraw);
        load_rows(vbase, b + 2, vraw);
        lds_barrier();
#pragma unroll
        for (int h = 0; h < H; h++)
#pragma unroll
            for (int kt = 0; kt < 2; kt++) { cur[h][kt] = next[h][kt]; }
    };
    for (int b = 0; b < n_plain; b++) { pass2_block(b, std::false_type{}); }
    for (int b = n_plain; b < n_blocks; b++) { pass2_block(b, std::true_type{}); }
    // the two key halves of a head group meet in LDS (the staging buffers are free now): lane-major, so that consecutive
    // lanes touch consecutive words
    float* red = (float*)&ks[0][0];
    static_assert(sizeof(ks) >= (size_t)(NW / 2) * H * 8 * 4 * 64 * sizeof(float), "reduction buffer");
    if (active && kh == 1)
    {
#pragma unroll
        for (int h = 0; h < H; h++)
#pragma unroll
            for (int d = 0; d < 8; d++)
#pragma unroll
                for (int v = 0; v < 4; v++) { red[(((hg * H + h) * 8 + d) * 4 + v) * 64 + lane] = out[h][d][v]; }
    }
    lds_barrier();
    if (!active || kh == 1) { return; }
    // D of the last product: lane (dim = 16 d + j, g) holds tokens 4 g .. 4 g + 3 of the tile
#pragma unroll
    for (int h = 0; h < H; h++)
#pragma unroll
        for (int d = 0; d < 8; d++)
        {
#pragma unroll
            for (int v = 0; v < 4; v++)
            {
                const int t = t0 + 4 * g + v;
                const float sum = out[h][d][v] + red[(((hg * H + h) * 8 + d) * 4 + v) * 64 + lane];
                if (t < n_tokens) { y[((size_t)t * n_q + head0 + h) * 128 + 16 * d + j] = (uint16_t)f32_to_bf16_bits(sum); }
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

// r = bf16(a + b) and y = rmsnorm(r) * w for rows of at most 4096 values (a multiple of 8): the residual add and the norm
// that follows it in one pass, with add_rows_kernel's rounding and rms_norm_rows_kernel's arithmetic (a wave per row, the
// row stays in registers, the same order of the sum of squares), so the pair gives the same bits as the two launches.
static __global__ __launch_bounds__(256) void add_rms_norm_rows_kernel(const uint16_t* __restrict__ A, const uint16_t* __restrict__ B, uint16_t* __restrict__ R,
                                                               const uint16_t* __restrict__ scale, uint16_t* __restrict__ Y, unsigned outer, unsigned inner, float eps)
{
    const unsigned lane = threadIdx.x & 63u;
    const unsigned row = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (row >= outer) { return; }
    const size_t base = (size_t)row * inner;
    const unsigned n_chunks = inner / 8u;                   // 16-byte chunks of the row; chunk c belongs to lane c % 64
    // every load is issued before the first use (a load inside a per-lane branch waits for the one before it); lanes past
    // the row's end re-read its last chunk and drop it
    u32x4 v[RMS_CHUNKS], va[RMS_CHUNKS], vb[RMS_CHUNKS], w[RMS_CHUNKS];
    const int n_j = n_chunks <= 64u ? 1 : RMS_CHUNKS;
#pragma unroll
    for (int j = 0; j < RMS_CHUNKS; j++)
    {
        if (j < n_j)
        {
            const unsigned c = min(lane + 64u * j, n_chunks - 1u);
            va[j] = *(const u32x4*)(A + base + c * 8u);
            vb[j] = *(const u32x4*)(B + base + c * 8u);
            w[j] = *(const u32x4*)(scale + c * 8u);
        }
    }
    float sumsq = 0.0f;
#pragma unroll
    for (int j = 0; j < RMS_CHUNKS; j++)
    {
        const unsigned c = lane + 64u * j;
        v[j] = u32x4{ 0u, 0u, 0u, 0u };
        if (j < n_j && c < n_chunks)
        {
#pragma unroll
            for (int d = 0; d < 4; d++)
            {
                const float lo = bf16_bits_to_f32(va[j][d] & 0xFFFFu) + bf16_bits_to_f32(vb[j][d] & 0xFFFFu);
                const float hi = bf16_bits_to_f32(va[j][d] >> 16) + bf16_bits_to_f32(vb[j][d] >> 16);
                v[j][d] = f32_to_bf16_bits(lo) | (f32_to_bf16_bits(hi) << 16);
            }
            *(u32x4*)(R + base + c * 8u) = v[j];
        }
        sumsq += sumsq8(v[j]);
    }
    const float invstd = rsqrtf(wave_sum(sumsq) / (float)inner + eps);
#pragma unroll
    for (int j = 0; j < RMS_CHUNKS; j++)
    {
        const unsigned c = lane + 64u * j;
        if (j < n_j && c < n_chunks) { *(u32x4*)(Y + base + c * 8u) = normed8(v[j], w[j], invstd); }
    }
}

}    // namespace ccq
