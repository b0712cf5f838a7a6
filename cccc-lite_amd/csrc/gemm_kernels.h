// Prefill GEMM for gfx950 (tokens > 16): weight tiles are dequantised to BF16 on their way into
// LDS and both operands feed v_mfma_f32_32x32x16_bf16 with FP32 accumulation; one rounding to
// BF16 in the epilogue.  Same numerics as the reference's dequantise-then-BF16-GEMM
// (cccc/cublas_real.h:943-964): the weight value entering a product is bf16(decode(w) * scale).
//
// Tiling: a 256-thread workgroup (4 waves, 2 x 2) owns BM output features x BN tokens and walks K
// in steps of BK (64 or 128).  LDS holds one X tile [BN][BK] and one dequantised W tile [BM][BK];
// the 16-byte chunks of a row are XOR-swizzled so that the 128-bit fragment reads of 16 consecutive
// rows hit 16 distinct bank groups.  The next k-tile is fetched from global memory into registers
// while the current one is multiplied.  With XCD = true, workgroup ids that are congruent mod 8
// (they land on the same XCD) walk the token tiles of one weight tile, so a weight tile is pulled
// from HBM once per XCD and shared through that XCD's L2.
//   A operand (rows)    = tokens,          lane (r = lane % 32, h = lane / 32) holds k = 8 h .. 8 h + 7
//   B operand (columns) = output features, same k split
//   D: lane holds column lane % 32; register v is row 8 (v / 4) + 4 (lane / 32) + v % 4
#pragma once
#include "gemv_kernels.h"
#include "linear_args.h"
#include "quant_device.h"
#include "runtime.h"
#include <type_traits>

namespace ccq
{

// LDS rows of CPR 16-byte chunks: 8 chunks (128-byte rows, two rows per 256-byte bank sweep) or
// 16 chunks (256-byte rows, every row starts at bank 0)
template <int CPR>
__device__ __forceinline__ int swizzled_chunk_n(int row, int chunk) { return CPR == 16 ? (chunk ^ (row & 15)) : (chunk ^ ((row >> 1) & 7)); }

// 16 FP8 codes -> 16 BF16 (two 16-byte LDS chunks)
template <int WT, bool SCALED, int AT = DT_BF16>
__device__ __forceinline__ void dequant16_fp8(const u32x4& w, float scale, u32x4& lo, u32x4& hi)
{
    uint32_t out[8];
#pragma unroll
    for (int d = 0; d < 4; d++)
    {
        typename ActPair<AT>::type p, q;
        fp8x4_to_pairs<WT, SCALED, AT>(w[d], scale, p, q);
        out[2 * d] = __builtin_bit_cast(uint32_t, p);
        out[2 * d + 1] = __builtin_bit_cast(uint32_t, q);
    }
    lo = u32x4{ out[0], out[1], out[2], out[3] };
    hi = u32x4{ out[4], out[5], out[6], out[7] };
}

// 8 FP4 codes (one dword) times a block scale -> 8 BF16 (one 16-byte LDS chunk)
__device__ __forceinline__ u32x4 dequant8_fp4(uint32_t w, float scale)
{
    uint32_t out[4];
#pragma unroll
    for (int b = 0; b < 4; b++)
    {
        f32x2 v;
        switch (b)
        {
        case 0: v = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 0); break;
        case 1: v = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 1); break;
        case 2: v = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 2); break;
        default: v = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 3); break;
        }
        const bf16x2 p = { (__bf16)(v.x * scale), (__bf16)(v.y * scale) };
        out[b] = __builtin_bit_cast(uint32_t, p);
    }
    return u32x4{ out[0], out[1], out[2], out[3] };
}

// WT: DT_E5M2 / DT_E4M3 / DT_FP4.  BLOCK: FP4 block length (16 / 32), unused for FP8.
// Requires K % 16 == 0 (FP8) or K % 32 == 0 (FP4), and the alignment rules of the GEMV kernels.
template <int WT, int BLOCK, int BM, int BN, bool SCALED, int BK = 64, bool XCD = false, int AT = DT_BF16>
__global__ __launch_bounds__(256) void gemm_mfma_kernel(const LinearArgs a, const int n_tiles, const int m_tiles)
{
    constexpr int WM = BM / 2;          // output features per wave
    constexpr int WN = BN / 2;          // tokens per wave
    constexpr int TM = WM / 32;         // MFMA tiles along output features
    constexpr int TN = WN / 32;         // MFMA tiles along tokens
    constexpr bool FP4 = WT == DT_FP4;
    constexpr int W_CHUNK_K = FP4 ? 32 : 16;                // elements per 16-byte global chunk
    constexpr int W_CHUNKS = BM * (BK / W_CHUNK_K);         // per k-tile
    constexpr int W_PER_THREAD = (W_CHUNKS + 255) / 256;
    constexpr int X_PER_THREAD = BN * (BK / 8) / 256;

    constexpr int CPR = BK / 8;                              // 16-byte BF16 chunks per LDS row
    __shared__ u32x4 xs[BN * CPR];
    __shared__ u32x4 ws[BM * CPR];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wave_m = wave & 1;
    const int wave_n = wave >> 1;
    int n_tile, m_tile;
    if (XCD)
    {
        // workgroups whose ids are congruent mod 8 share an XCD: let them walk the token tiles of one weight tile
        const int seq = blockIdx.x >> 3;
        n_tile = (blockIdx.x & 7) + 8 * (seq / m_tiles);
        m_tile = seq % m_tiles;
        if (n_tile >= n_tiles) { return; }
    }
    else
    {
        n_tile = blockIdx.x % n_tiles;
        m_tile = blockIdx.x / n_tiles;
    }
    const int out_base = n_tile * BM;
    const int tok_base = m_tile * BN;

    f32x16 acc[TN][TM];
#pragma unroll
    for (int tn = 0; tn < TN; tn++)
#pragma unroll
        for (int tm = 0; tm < TM; tm++)
#pragma unroll
            for (int v = 0; v < 16; v++) { acc[tn][tm][v] = 0.0f; }

    u32x4 wreg[W_PER_THREAD];
    uint32_t sreg[W_PER_THREAD];
    u32x4 xreg[X_PER_THREAD];

    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < W_PER_THREAD; i++)
        {
            const int q = tid + i * 256;
            const int row_in_tile = q / (BK / W_CHUNK_K);
            const int part = q % (BK / W_CHUNK_K);
            const int k = k0 + part * W_CHUNK_K;
            wreg[i] = u32x4{ 0u, 0u, 0u, 0u };
            sreg[i] = 0u;
            if (q < W_CHUNKS && k < a.K)
            {
                const long long row = min(out_base + row_in_tile, a.n_out - 1);
                const long long flat = row * a.ldw + k;
                wreg[i] = *(const u32x4*)(a.W + (FP4 ? (flat >> 1) : flat));
                if (FP4)
                {
                    if (BLOCK == 16) { sreg[i] = *(const uint16_t*)(a.blk_sc + flat / 16); }
                    else { sreg[i] = a.blk_sc[flat / 32]; }
                }
            }
        }
#pragma unroll
        for (int i = 0; i < X_PER_THREAD; i++)
        {
            const int q = tid + i * 256;
            const int row_in_tile = q / CPR;
            const int chunk = q % CPR;
            const int k = k0 + chunk * 8;
            xreg[i] = u32x4{ 0u, 0u, 0u, 0u };
            if (k < a.K)
            {
                const long long tok = min(tok_base + row_in_tile, a.tokens - 1);
                xreg[i] = *(const u32x4*)(a.X + tok * a.ldx + k);
            }
        }
    };

    auto stage = [&]() {
#pragma unroll
        for (int i = 0; i < W_PER_THREAD; i++)
        {
            const int q = tid + i * 256;
            if (q < W_CHUNKS)
            {
                const int row = q / (BK / W_CHUNK_K);
                const int part = q % (BK / W_CHUNK_K);
                if (FP4)
                {
                    const float s0 = __builtin_amdgcn_cvt_f32_fp8(sreg[i], 0);
                    const float s1 = BLOCK == 16 ? __builtin_amdgcn_cvt_f32_fp8(sreg[i], 1) : s0;
#pragma unroll
                    for (int d = 0; d < 4; d++)
                    {
                        ws[row * CPR + swizzled_chunk_n<CPR>(row, part * 4 + d)] = dequant8_fp4(wreg[i][d], d < 2 ? s0 : s1);
                    }
                }
                else
                {
                    u32x4 lo, hi;
                    dequant16_fp8<WT, SCALED, AT>(wreg[i], a.w_scale, lo, hi);
                    ws[row * CPR + swizzled_chunk_n<CPR>(row, part * 2)] = lo;
                    ws[row * CPR + swizzled_chunk_n<CPR>(row, part * 2 + 1)] = hi;
                }
            }
        }
#pragma unroll
        for (int i = 0; i < X_PER_THREAD; i++)
        {
            const int q = tid + i * 256;
            const int row = q / CPR;
            xs[row * CPR + swizzled_chunk_n<CPR>(row, q % CPR)] = xreg[i];
        }
    };

    const int r32 = lane & 31;
    const int h = lane >> 5;

    fetch(0);
    for (int k0 = 0; k0 < a.K; k0 += BK)
    {
        stage();
        __syncthreads();
        if (k0 + BK < a.K) { fetch(k0 + BK); }
#pragma unroll
        for (int ks = 0; ks < BK / 16; ks++)
        {
            typedef typename std::conditional<AT == DT_HALF, f16x8, bf16x8>::type frag_t;
            frag_t xf[TN], wf[TM];
#pragma unroll
            for (int tn = 0; tn < TN; tn++)
            {
                const int row = wave_n * WN + tn * 32 + r32;
                xf[tn] = __builtin_bit_cast(frag_t, xs[row * CPR + swizzled_chunk_n<CPR>(row, ks * 2 + h)]);
            }
#pragma unroll
            for (int tm = 0; tm < TM; tm++)
            {
                const int row = wave_m * WM + tm * 32 + r32;
                wf[tm] = __builtin_bit_cast(frag_t, ws[row * CPR + swizzled_chunk_n<CPR>(row, ks * 2 + h)]);
            }
#pragma unroll
            for (int tn = 0; tn < TN; tn++)
#pragma unroll
                for (int tm = 0; tm < TM; tm++)
                {
                    if constexpr (AT == DT_HALF) { acc[tn][tm] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xf[tn], wf[tm], acc[tn][tm], 0, 0, 0); }
                    else { acc[tn][tm] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xf[tn], wf[tm], acc[tn][tm], 0, 0, 0); }
                }
        }
        __syncthreads();
    }

#pragma unroll
    for (int tn = 0; tn < TN; tn++)
    {
#pragma unroll
        for (int tm = 0; tm < TM; tm++)
        {
            const int out = out_base + wave_m * WM + tm * 32 + r32;
#pragma unroll
            for (int v = 0; v < 16; v++)
            {
                const int tok = tok_base + wave_n * WN + tn * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
                if (out < a.n_out && tok < a.tokens)
                {
                    uint16_t* y = a.Y + (long long)tok * a.y_stride_tok + (long long)out * a.y_stride_out;
                    *y = finish_output_act<AT>(acc[tn][tm][v], a.alpha, a.beta, y);
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// FP8 GEMM whose weights never pass through LDS.  A workgroup of four waves owns MB * 16 tokens x
// 256 output features; wave w owns features 64 w .. 64 w + 63 for all of the tokens.  Each lane
// loads the 16 weight bytes it will feed to the matrix cores itself -- row (lane % 16) of a 16-row
// block, bytes 16 (lane / 16) .. + 15 of the 64-byte k-tile -- and converts them in registers: the
// low 8 bytes are its row operand of the first v_mfma_f32_16x16x32 of the k-tile and the high 8 bytes
// that of the second.  The contraction does not care in which order k is visited as long as both
// operands agree, so the token operand is read from LDS with the matching k assignment (chunk
// 2 (lane / 16) + step of the row).  Only the activations are staged through LDS (one 128-byte row
// per token and k-tile, XOR-swizzled, two buffers, one barrier per k-tile); per matrix-core
// instruction the LDS then moves a quarter of the bytes the two-operand kernel above needs.
//   A operand (rows)    = features: lane (i = lane % 16, g = lane / 16) holds k = 16 g + 8 step .. + 7
//   B operand (columns) = tokens:   same k
//   D: lane holds token lane % 16; register v is feature 4 (lane / 16) + v, so a lane ends with four
//      consecutive outputs of one token row (one 8-byte store)
// SPLIT: blockIdx.y selects one of gridDim.y equal ranges of k-tiles; the FP32 partial sums of range s go
// to partial[s][token][feature] (no alpha / beta) and gemm_splitk_combine_kernel finishes them.  Used when
// the output has too few tiles to fill the machine.
// NB: 16-feature blocks per wave (a workgroup owns 64 NB features): 4 by default; 3 or 2 give the launch more, smaller
// workgroups when the output has too few 256-feature tiles to fill the machine evenly.
// PAIR: two weights of one shape (a.W = gate, a.W_pair = up) against the same activations; a wave's first NB / 2 feature
// blocks are gate rows, the other NB / 2 the same rows of up, and the epilogue writes the reference's SwiGLU product
// bf16(bf16(g * bf16(sigmoid g)) * u) of the two rounded linears (cccc/MatrixEx.cpp:756-762, hip_functions.cpp:722-732,
// :953-966) -- one launch instead of two GEMMs and an elementwise pass over three [tokens][n_out] matrices.  A workgroup
// then owns 32 NB output features; alpha = 1, beta = 0, BF16.
// SEG: the launch covers up to three linears on the same activations (the q, k and v projections: the narrow ones alone
// leave most CUs idle); a workgroup finds its segment from its feature tile and takes that segment's weight, output,
// width and scale -- from there on it is the single-linear kernel.
// PD: how many k-tiles ahead the weights are requested (the activations PD + 1 when PD > 1).  One is enough where two
// workgroups share a CU and each k-tile carries 64 matrix-core instructions per wave; the k-split launches of a short
// prompt (one 64-token tile, about one workgroup per CU) are bound by their weight bytes and run a k-tile per memory
// latency with PD = 1 -- they take PD = 3.
template <int WT, bool SCALED, int MB, bool SPLIT, bool TILED, int AT = DT_BF16, int NB = 4, bool PAIR = false, bool SEG = false, int PD = 1, int WGS_PER_CU = 2>
__global__ __launch_bounds__(256, WGS_PER_CU) void gemm_mfma_direct_kernel(const LinearArgs a_in, const int n_tiles, float* __restrict__ partial)
{
    static_assert(!PAIR || (NB % 2 == 0 && AT == DT_BF16), "pair: an even number of feature blocks, BF16");
    static_assert(!SEG || !PAIR, "segments: single linears");
    constexpr int NBO = PAIR ? NB / 2 : NB;     // feature blocks of a wave in the output
    constexpr int BTOK = MB * 16;               // tokens per workgroup
    constexpr int BK = 64, CPR = 8;
    constexpr int X_PER_THREAD = BTOK * CPR / 256;
    __shared__ u32x4 xs[2][BTOK * CPR];
    typedef typename std::conditional<AT == DT_HALF, f16x8, bf16x8>::type frag_t;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // The hardware hands consecutive workgroups to the eight XCDs in turn, each with an L2 of its own.  With the feature
    // tiles padded to a multiple of eight, feature tile n always lands on XCD n % 8, and the workgroups an XCD runs at
    // one time are a block of (n_pad / 8) feature tiles x several token tiles: both operands are shared inside the L2.
    const int n_pad = (n_tiles + 7) & ~7;
    int n_tile = blockIdx.x % n_pad;
    const int m_tile = blockIdx.x / n_pad;
    if (n_tile >= n_tiles) { return; }          // padding
    LinearArgs a = a_in;
    if constexpr (SEG)
    {
        const int s = n_tile >= a_in.seg_tile0[2] ? 2 : (n_tile >= a_in.seg_tile0[1] ? 1 : 0);
        a.W = a_in.seg_W[s];
        a.Y = a_in.seg_Y[s];
        a.n_out = a_in.seg_n_out[s];
        a.w_scale = a_in.seg_w_scale[s];
        a.y_stride_tok = a_in.seg_y_stride_tok[s];
        n_tile -= a_in.seg_tile0[s];
        // the partial sums of a segment follow those of the segments before it
        if constexpr (SPLIT) { partial += (long long)gridDim.y * a_in.tokens * ((s > 0 ? a_in.seg_n_out[0] : 0) + (s > 1 ? a_in.seg_n_out[1] : 0)); }
    }
    const int out_base = n_tile * (64 * NBO) + wave * (16 * NBO);
    const int tok_base = m_tile * BTOK;
    const int i16 = lane & 15;
    const int g = lane >> 4;
    const int n_kt_total = a.K / BK;
    const int kt_begin = SPLIT ? (int)((long long)n_kt_total * blockIdx.y / gridDim.y) : 0;
    const int n_kt = SPLIT ? (int)((long long)n_kt_total * (blockIdx.y + 1) / gridDim.y) - kt_begin : n_kt_total;
    const uint8_t* const w_begin = a.W + (long long)kt_begin * (TILED ? 1024 : BK);
    const uint8_t* const x_begin = (const uint8_t*)a.X + (long long)kt_begin * BK * 2;

    f32x4 acc[MB][NB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++) { acc[mb][nb] = f32x4{ 0.0f, 0.0f, 0.0f, 0.0f }; }

    // Every address in the loop is a wave-uniform base (scalar registers, advanced by scalar adds) plus a
    // 32-bit per-lane byte offset fixed for the whole kernel; the launcher checks that both operands are
    // smaller than 4 GiB.
    // TILED: a.W is the repacked copy (repack_tiled_kernel), where the KiB one load instruction of a wave
    // takes -- 16 rows x 64 codes -- is contiguous and the next k-tile follows it.
    long long w_tile_base[NB];
    uint32_t w_off[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
    {
        const int ob = nb % NBO;                            // feature block within the wave's output
        if (TILED)
        {
            w_tile_base[nb] = (long long)min(out_base / 16 + ob, (a.n_out + 15) / 16 - 1) * n_kt_total * 1024;
            w_off[nb] = lane * 16;
        }
        else
        {
            w_tile_base[nb] = 0;
            w_off[nb] = (uint32_t)((long long)min(out_base + ob * 16 + i16, a.n_out - 1) * a.ldw + g * 16);
        }
        if (PAIR && nb >= NBO) { w_tile_base[nb] += (long long)((intptr_t)a.W_pair - (intptr_t)a.W); }      // the up weight, addressed from the gate weight's base
    }
    uint32_t x_off[X_PER_THREAD];
#pragma unroll
    for (int i = 0; i < X_PER_THREAD; i++)
    {
        const int q = tid + i * 256;
        x_off[i] = (uint32_t)(((long long)min(tok_base + q / CPR, a.tokens - 1) * a.ldx + (q % CPR) * 8) * 2);
    }
    // LDS slots: where this thread stores its activation chunks, and where it reads its A operands
    int x_store[X_PER_THREAD];
#pragma unroll
    for (int i = 0; i < X_PER_THREAD; i++)
    {
        const int q = tid + i * 256;
        x_store[i] = (q / CPR) * CPR + swizzled_chunk_n<CPR>(q / CPR, q % CPR);
    }

    constexpr int RW = PD + 1;                  // weight register buffers: tile kt lives in wraw[kt % RW]
    constexpr int RX = PD == 1 ? 1 : PD + 1;    // activation register buffers: tile kt travels in xring[kt % RX]
    u32x4 wraw[RW][NB], xring[RX][X_PER_THREAD];
    // K is a multiple of 64 here and the k-tile index of a prefetch is clamped to the last one, so no load
    // or store in the loop needs a predicate or a branch: the wait counts stay exact
    auto fetch_x = [&](int kt, u32x4* xreg) {
        const int k0 = min(kt, n_kt - 1) * BK;
#pragma unroll
        for (int i = 0; i < X_PER_THREAD; i++) { xreg[i] = *(const u32x4*)(x_begin + (size_t)k0 * 2 + (size_t)x_off[i]); }
    };
    auto fetch_w = [&](int kt, u32x4* wraw) {
        const int k0 = min(kt, n_kt - 1) * (TILED ? 1024 : BK);
#pragma unroll
        for (int nb = 0; nb < NB; nb++) { wraw[nb] = *(const u32x4*)(w_begin + w_tile_base[nb] + k0 + (size_t)w_off[nb]); }
    };
    auto stage = [&](int buf, const u32x4* xreg) {
#pragma unroll
        for (int i = 0; i < X_PER_THREAD; i++) { xs[buf][x_store[i]] = xreg[i]; }
    };

    // Order of one k-tile: barrier | the matrix-core work, token block by token block, with one memory instruction in
    // front of each block: the NB weight pieces of tile kt + PD with the first blocks, from the middle on the stores of
    // the next activation tile to LDS, each followed one block later by the load that refills its register.  The LDS
    // stores and the global loads are thus a whole k-tile of work away from the instructions that wait for them, nothing
    // but the barrier and the first fragment read stands between two k-tiles, and no burst of memory instructions holds
    // up the fragment reads queued behind it (all of them in one place each: 1-3 % slower on the benchmark shapes).
    // wcur: tile kt; wnext: the buffer tile kt + PD goes to; xreg: tile kt + 1, replaced by tile kt + 1 + RX.
    auto k_tile = [&](int kt, u32x4* wcur, u32x4* wnext, u32x4* xreg) {
        u32x4 wf[2][NB];
#pragma unroll
        for (int nb = 0; nb < NB; nb++) { dequant16_fp8<WT, SCALED, AT>(wcur[nb], PAIR && nb >= NBO ? a.w_scale_pair : a.w_scale, wf[0][nb], wf[1][nb]); }
        if constexpr (PD == 1) { __syncthreads(); }          // tile kt is in xs[kt & 1]; the other buffer is free
        else { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }    // LDS order only: the loads of later tiles stay in flight
        const int w_k0 = min(kt + PD, n_kt - 1) * (TILED ? 1024 : BK);
        const int x_k0 = min(kt + 1 + RX, n_kt - 1) * BK;
        const u32x4* xt = xs[kt & 1];
        // token fragments run AHEAD instructions in front of the matrix-core instructions that use them
        constexpr int AHEAD = 3, FRAGS = 2 * MB;
        auto read_frag = [&](int f) {
            const int row = (f % MB) * 16 + i16;
            return xt[row * CPR + swizzled_chunk_n<CPR>(row, 2 * g + f / MB)];
        };
        u32x4 ring[AHEAD + 1];
#pragma unroll
        for (int f = 0; f < AHEAD; f++) { ring[f] = read_frag(f); }
        static_assert(NB <= FRAGS && FRAGS / 2 + 1 + X_PER_THREAD <= FRAGS, "one slot per memory instruction");
#pragma unroll
        for (int f = 0; f < FRAGS; f++)
        {
            if (f < NB) { wnext[f] = *(const u32x4*)(w_begin + w_tile_base[f] + w_k0 + (size_t)w_off[f]); }
            if (f >= FRAGS / 2 && f < FRAGS / 2 + X_PER_THREAD) { xs[(kt + 1) & 1][x_store[f - FRAGS / 2]] = xreg[f - FRAGS / 2]; }
            if (f >= FRAGS / 2 + 1 && f < FRAGS / 2 + 1 + X_PER_THREAD)
            {
                const int i = f - FRAGS / 2 - 1;
                xreg[i] = *(const u32x4*)(x_begin + (size_t)x_k0 * 2 + (size_t)x_off[i]);
            }
            if (f + AHEAD < FRAGS) { ring[(f + AHEAD) % (AHEAD + 1)] = read_frag(f + AHEAD); }
            const frag_t xf = __builtin_bit_cast(frag_t, ring[f % (AHEAD + 1)]);
            const int s = f / MB, mb = f % MB;
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
            {
                const frag_t w = __builtin_bit_cast(frag_t, wf[s][nb]);
                if constexpr (AT == DT_HALF) { acc[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w, xf, acc[mb][nb], 0, 0, 0); }
                else { acc[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w, xf, acc[mb][nb], 0, 0, 0); }
            }
        }
        // pin the order: the scheduler otherwise pulls every read down to just before its first use
        __builtin_amdgcn_sched_group_barrier(0x100, AHEAD, 0);
#pragma unroll
        for (int f = 0; f < FRAGS; f++)
        {
            if (f < NB) { __builtin_amdgcn_sched_group_barrier(0x020, 1, 0); }
            if (f >= FRAGS / 2 && f < FRAGS / 2 + X_PER_THREAD) { __builtin_amdgcn_sched_group_barrier(0x200, 1, 0); }
            if (f >= FRAGS / 2 + 1 && f < FRAGS / 2 + 1 + X_PER_THREAD) { __builtin_amdgcn_sched_group_barrier(0x020, 1, 0); }
            if (f + AHEAD < FRAGS) { __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); }
            __builtin_amdgcn_sched_group_barrier(0x008, NB, 0);
        }
    };

    fetch_x(0, xring[0]);
#pragma unroll
    for (int t = 0; t < PD; t++) { fetch_w(t, wraw[t]); }
    stage(0, xring[0]);
#pragma unroll
    for (int t = 1; t <= RX; t++) { fetch_x(t, xring[t % RX]); }
    if constexpr (PD == 1)
    {
        for (int kt = 0; kt < n_kt; kt += 2)
        {
            k_tile(kt, wraw[0], wraw[1], xring[0]);
            if (kt + 1 < n_kt) { k_tile(kt + 1, wraw[1], wraw[0], xring[0]); }
        }
    }
    else
    {
        // whole rounds of the register ring without a branch between the tiles (behind a skipped tile the compiler has to
        // assume that fewer loads are in flight and waits for all but a few), then the last 0 .. PD tiles
        int kt = 0;
        for (; kt + RW <= n_kt; kt += RW)
        {
#pragma unroll
            for (int j = 0; j < RW; j++) { k_tile(kt + j, wraw[j], wraw[(j + PD) % RW], xring[(j + 1) % RX]); }
        }
#pragma unroll
        for (int j = 0; j < PD; j++)
        {
            if (kt + j < n_kt) { k_tile(kt + j, wraw[j], wraw[(j + PD) % RW], xring[(j + 1) % RX]); }
        }
    }

    const bool wide_store = SPLIT ? a.n_out % 4 == 0 : (a.y_stride_out == 1 && a.y_stride_tok % 4 == 0 && ((uintptr_t)a.Y & 7u) == 0);
    if constexpr (PAIR && !SPLIT)
    {
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
        {
            const int tok = tok_base + mb * 16 + i16;
            if (tok >= a.tokens) { continue; }
#pragma unroll
            for (int nb = 0; nb < NBO; nb++)
            {
                const int out = out_base + nb * 16 + 4 * g;
                if (out >= a.n_out) { continue; }
                uint16_t o[4];
#pragma unroll
                for (int v = 0; v < 4; v++)
                {
                    const float gate = bf16_bits_to_f32(f32_to_bf16_bits(acc[mb][nb][v])), up = bf16_bits_to_f32(f32_to_bf16_bits(acc[mb][nb + NBO][v]));
                    const float sig = bf16_bits_to_f32(f32_to_bf16_bits(1.0f / (1.0f + expf(-gate))));
                    o[v] = (uint16_t)f32_to_bf16_bits(bf16_bits_to_f32(f32_to_bf16_bits(gate * sig)) * up);
                }
                uint16_t* y = a.Y + (long long)tok * a.y_stride_tok + (long long)out * a.y_stride_out;
                if (wide_store && out + 3 < a.n_out) { *(uint2*)y = uint2{ (uint32_t)o[0] | ((uint32_t)o[1] << 16), (uint32_t)o[2] | ((uint32_t)o[3] << 16) }; }
                else
                {
#pragma unroll
                    for (int v = 0; v < 4; v++)
                    {
                        if (out + v < a.n_out) { y[v * a.y_stride_out] = o[v]; }
                    }
                }
            }
        }
        return;
    }
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
    {
        const int tok = tok_base + mb * 16 + i16;
        if (tok >= a.tokens) { continue; }
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
        {
            const int out = out_base + (nb % NBO) * 16 + 4 * g;
            if (out >= a.n_out) { continue; }
            const f32x4 r = acc[mb][nb];
            if constexpr (SPLIT)
            {
                // pair: the up weight's sums are a second set behind all of the gate weight's
                float* p = partial + (((long long)(nb / NBO) * gridDim.y + blockIdx.y) * a.tokens + tok) * a.n_out + out;
                if (wide_store && out + 3 < a.n_out) { *(f32x4*)p = r; }
                else
                {
#pragma unroll
                    for (int v = 0; v < 4; v++)
                    {
                        if (out + v < a.n_out) { p[v] = r[v]; }
                    }
                }
            }
            else
            {
                uint16_t* y = a.Y + (long long)tok * a.y_stride_tok + (long long)out * a.y_stride_out;
                if (wide_store && out + 3 < a.n_out)
                {
                    uint16_t old[4] = { 0, 0, 0, 0 };
                    if (a.beta != 0.0f) { *(uint2*)old = *(const uint2*)y; }
                    uint16_t o[4];
#pragma unroll
                    for (int v = 0; v < 4; v++) { o[v] = finish_output_act<AT>(r[v], a.alpha, a.beta, &old[v]); }
                    *(uint2*)y = uint2{ (uint32_t)o[0] | ((uint32_t)o[1] << 16), (uint32_t)o[2] | ((uint32_t)o[3] << 16) };
                }
                else
                {
#pragma unroll
                    for (int v = 0; v < 4; v++)
                    {
                        if (out + v < a.n_out) { y[v * a.y_stride_out] = finish_output_act<AT>(r[v], a.alpha, a.beta, y + v * a.y_stride_out); }
                    }
                }
            }
        }
    }
}

// Sums the FP32 partial tiles of a k-split GEMM and applies alpha / beta and the one rounding.  One thread
// per four consecutive features of a token (n_out is a multiple of 4 on this path).
// SEG: the partial sums of up to three linears, each laid out as its own k-split GEMM, one after the other; a thread finds
// its segment from its feature.  PAIR: gate sums, then up sums; the thread adds both and writes the SwiGLU product with the
// roundings of the unsplit pair kernel's epilogue.
template <int AT, bool SEG = false, bool PAIR = false>
__global__ __launch_bounds__(256) void gemm_splitk_combine_kernel(const float* __restrict__ partial, const int splits, const LinearArgs a_in)
{
    LinearArgs a = a_in;
    const int n_all = SEG ? a_in.seg_n_out[0] + a_in.seg_n_out[1] + a_in.seg_n_out[2] : a_in.n_out;
    const long long groups = (long long)a.tokens * (n_all / 4);
    for (long long q = (long long)blockIdx.x * 256 + threadIdx.x; q < groups; q += (long long)gridDim.x * 256)
    {
        const int tok = (int)(q / (n_all / 4));
        int out = (int)(q % (n_all / 4)) * 4;
        const float* p = partial;
        if constexpr (SEG)
        {
            const int n0 = a_in.seg_n_out[0], n01 = n0 + a_in.seg_n_out[1];
            const int s = out >= n01 ? 2 : (out >= n0 ? 1 : 0);
            const int start = s == 2 ? n01 : (s == 1 ? n0 : 0);
            a.Y = a_in.seg_Y[s];
            a.n_out = a_in.seg_n_out[s];
            a.y_stride_tok = a_in.seg_y_stride_tok[s];
            p += (long long)splits * a.tokens * start;
            out -= start;
        }
        const long long slice = (long long)a.tokens * a.n_out;
        p += (long long)tok * a.n_out + out;
        f32x4 r = *(const f32x4*)p;
        for (int s = 1; s < splits; s++) { r += *(const f32x4*)(p + s * slice); }
        const bool wide_store = a.y_stride_out == 1 && a.y_stride_tok % 4 == 0 && ((uintptr_t)a.Y & 7u) == 0;
        uint16_t* y = a.Y + (long long)tok * a.y_stride_tok + (long long)out * a.y_stride_out;
        if constexpr (PAIR)
        {
            const float* pu = p + splits * slice;
            f32x4 u = *(const f32x4*)pu;
            for (int s = 1; s < splits; s++) { u += *(const f32x4*)(pu + s * slice); }
            uint16_t o[4];
#pragma unroll
            for (int v = 0; v < 4; v++)
            {
                const float gate = bf16_bits_to_f32(f32_to_bf16_bits(r[v])), up = bf16_bits_to_f32(f32_to_bf16_bits(u[v]));
                const float sig = bf16_bits_to_f32(f32_to_bf16_bits(1.0f / (1.0f + expf(-gate))));
                o[v] = (uint16_t)f32_to_bf16_bits(bf16_bits_to_f32(f32_to_bf16_bits(gate * sig)) * up);
            }
            if (wide_store) { *(uint2*)y = uint2{ (uint32_t)o[0] | ((uint32_t)o[1] << 16), (uint32_t)o[2] | ((uint32_t)o[3] << 16) }; }
            else
            {
#pragma unroll
                for (int v = 0; v < 4; v++) { y[v * a.y_stride_out] = o[v]; }
            }
            continue;
        }
        if (wide_store)
        {
            uint16_t old[4] = { 0, 0, 0, 0 };
            if (a.beta != 0.0f) { *(uint2*)old = *(const uint2*)y; }
            uint16_t o[4];
#pragma unroll
            for (int v = 0; v < 4; v++) { o[v] = finish_output_act<AT>(r[v], a.alpha, a.beta, &old[v]); }
            *(uint2*)y = uint2{ (uint32_t)o[0] | ((uint32_t)o[1] << 16), (uint32_t)o[2] | ((uint32_t)o[3] << 16) };
        }
        else
        {
#pragma unroll
            for (int v = 0; v < 4; v++) { y[v * a.y_stride_out] = finish_output_act<AT>(r[v], a.alpha, a.beta, y + v * a.y_stride_out); }
        }
    }
}

// ------------------------------------------------------------------------------------------
// The same GEMM for FP4 block-scale weights, on their load-time tiled copy (repack_tiled_fp4_kernel): per 16-row tile and
// 128-element chunk one contiguous KiB of codes -- lane (n = lane % 16, g = lane / 16) owns 16 bytes whose dword d holds
// row n's elements 32 d + 4 g .. + 3 (low 16 bits) and 32 d + 16 + 4 g .. + 3 (high 16 bits) of the chunk -- and, behind
// all code KiBs, 128 / BLOCK scale bytes per row and chunk.  One dword is therefore the lane's row operand of one
// v_mfma_f32_16x16x32_bf16 (k = those eight elements), dwords 0, 1 belong to the first 64-element half of the chunk and
// 2, 3 to the second.  fp4 * e4m3 has at most six significant bits, so bf16(fp4 * s) is exact: the codes are converted
// to FP32 (v_cvt_scalef32_pk_f32_fp4; the hardware conversion itself only applies a power-of-two scale), multiplied by
// the block scale and packed to BF16 in registers -- 16 VALU instructions per dword, shared by the MB token blocks.
// The activation tile of a 64-element half is staged in LDS already in that operand order: 16-byte piece 4 s + g of a
// token row holds elements 32 s + 4 g .. + 3 and 32 s + 16 + 4 g .. + 3, so a fragment is one 16-byte read.
// K % 128 == 0.  Tile shapes, k split and epilogue as in gemm_mfma_direct_kernel, except that the 128-token x 256-feature
// tile is compiled for one workgroup per CU (its accumulators, two operand buffers and two raw chunks do not fit the
// 256 registers a wave has when two workgroups share a CU; with the whole register file the accumulators sit in AGPRs).
template <int BLOCK>
__device__ __forceinline__ u32x4 dequant8_fp4_blocks(uint32_t w, float s_lo, float s_hi)
{
    uint32_t out[4];
#pragma unroll
    for (int b = 0; b < 4; b++)
    {
        f32x2 v;
        switch (b)
        {
        case 0: v = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 0); break;
        case 1: v = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 1); break;
        case 2: v = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 2); break;
        default: v = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 3); break;
        }
        const float sc = (BLOCK == 16 && b >= 2) ? s_hi : s_lo;
        const bf16x2 p = { (__bf16)(v.x * sc), (__bf16)(v.y * sc) };
        out[b] = __builtin_bit_cast(uint32_t, p);
    }
    return u32x4{ out[0], out[1], out[2], out[3] };
}

// SEG: as in gemm_mfma_direct_kernel -- up to three linears on the same activations, a workgroup takes weight, scales,
// output and width of the segment its feature tile belongs to (a.seg_W[s] = tiled codes with the scales behind them).
// PAIR: as in the FP8 kernel -- a.W = gate, a.W_pair = up, two tiled copies of one shape (so the up weight's codes and scale
// bytes sit at the same offsets behind a.W_pair as the gate's behind a.W); a wave's first NB / 2 feature blocks are gate
// rows, the others the same rows of up; SwiGLU product in the epilogue, or in the combine launch when the k range is split.
template <int BLOCK, int MB, bool SPLIT, int NB = 4, bool SEG = false, bool PAIR = false, bool MEM_BURSTS = false>
__global__ __launch_bounds__(256, (MB * NB >= 32) ? 1 : 2) void gemm4_mfma_direct_kernel(const LinearArgs a_in, const uint8_t* scales_in, const int n_tiles,
                                                                                        float* __restrict__ partial)
{
    static_assert(BLOCK == 16 || BLOCK == 32, "block scale length");
    static_assert(!PAIR || (NB % 2 == 0 && !SEG), "pair: an even number of feature blocks, one pair of weights");
    constexpr int NBO = PAIR ? NB / 2 : NB;     // feature blocks of a wave in the output
    constexpr int NS = 128 / BLOCK;             // scale bytes per row and chunk
    constexpr int BTOK = MB * 16;
    constexpr int BK = 64, CPR = 8;
    constexpr int X_PER_THREAD = BTOK * CPR / 256;
    __shared__ u32x4 xs[2][BTOK * CPR];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // The hardware hands consecutive workgroups to the eight XCDs in turn, each with an L2 of its own.  With the feature
    // tiles padded to a multiple of eight, feature tile n always lands on XCD n % 8, and the workgroups an XCD runs at
    // one time are a block of (n_pad / 8) feature tiles x several token tiles: both operands are shared inside the L2.
    const int n_pad = (n_tiles + 7) & ~7;
    int n_tile = blockIdx.x % n_pad;
    const int m_tile = blockIdx.x / n_pad;
    if (n_tile >= n_tiles) { return; }          // padding
    LinearArgs a = a_in;
    const uint8_t* tiled_scales = scales_in;
    if constexpr (SEG)
    {
        const int s = n_tile >= a_in.seg_tile0[2] ? 2 : (n_tile >= a_in.seg_tile0[1] ? 1 : 0);
        a.W = a_in.seg_W[s];
        a.Y = a_in.seg_Y[s];
        a.n_out = a_in.seg_n_out[s];
        a.y_stride_tok = a_in.seg_y_stride_tok[s];
        tiled_scales = a.W + (long long)((a.n_out + 15) / 16) * (a.K / 128) * 1024;
        n_tile -= a_in.seg_tile0[s];
        // the partial sums of a segment follow those of the segments before it
        if constexpr (SPLIT) { partial += (long long)gridDim.y * a_in.tokens * ((s > 0 ? a_in.seg_n_out[0] : 0) + (s > 1 ? a_in.seg_n_out[1] : 0)); }
    }
    const int out_base = n_tile * (64 * NBO) + wave * (16 * NBO);
    const int tok_base = m_tile * BTOK;
    const int i16 = lane & 15;
    const int g = lane >> 4;
    const int chunks_total = a.K / 128;
    const int c_begin = SPLIT ? (int)((long long)chunks_total * blockIdx.y / gridDim.y) : 0;
    const int n_chunks = SPLIT ? (int)((long long)chunks_total * (blockIdx.y + 1) / gridDim.y) - c_begin : chunks_total;
    const int n_kt = 2 * n_chunks;
    const uint8_t* const x_begin = (const uint8_t*)a.X + (long long)c_begin * 128 * 2;

    f32x4 acc[MB][NB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++) { acc[mb][nb] = f32x4{ 0.0f, 0.0f, 0.0f, 0.0f }; }

    // Every address in the loop is a wave-uniform base (scalar registers) plus a 32-bit per-lane byte offset fixed for
    // the whole kernel.
    long long w_base[NB], s_base[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
    {
        const long long tile = min(out_base / 16 + nb % NBO, (a.n_out + 15) / 16 - 1);     // a clamped tile is computed and dropped
        w_base[nb] = (tile * chunks_total + c_begin) * 1024;
        s_base[nb] = (tile * chunks_total + c_begin) * (16 * NS);
        if (PAIR && nb >= NBO)
        {
            const long long up = (long long)((intptr_t)a.W_pair - (intptr_t)a.W);     // the up copy, addressed from the gate copy
            w_base[nb] += up;
            s_base[nb] += up;
        }
    }
    const uint32_t w_off = lane * 16, s_off = i16 * NS;
    uint32_t x_off[X_PER_THREAD];
#pragma unroll
    for (int i = 0; i < X_PER_THREAD; i++)
    {
        const int q = tid + i * 256;
        x_off[i] = (uint32_t)(((long long)min(tok_base + q / CPR, a.tokens - 1) * a.ldx + (q % CPR) * 8) * 2);
    }
    // LDS slot (in 8-byte units) of this thread's first activation piece: elements 8 q8 .. + 3 go to piece 4 s + g0 at
    // half hb, elements 8 q8 + 4 .. + 7 to piece 4 s + g0 + 1 (g0 is even, so that is the slot with bit 1 flipped); the
    // thread's further pieces are 32 rows apart, which leaves the swizzle unchanged
    int x_store;
    {
        const int row = tid / CPR, q8 = tid % CPR;
        const int st = q8 >> 2, hb = (q8 >> 1) & 1, g0 = 2 * (q8 & 1);
        x_store = (row * CPR + swizzled_chunk_n<CPR>(row, 4 * st + g0)) * 2 + hb;
    }

    u32x4 wraw_a[NB], wraw_b[NB], xreg[X_PER_THREAD];
    u32x2 sraw_a[NB], sraw_b[NB];
    auto fetch_x = [&](int kt) {
        const int k0 = min(kt, n_kt - 1) * BK;
#pragma unroll
        for (int i = 0; i < X_PER_THREAD; i++) { xreg[i] = *(const u32x4*)(x_begin + (size_t)k0 * 2 + (size_t)x_off[i]); }
    };
    auto fetch_w = [&](int c, u32x4* wraw, u32x2* sraw) {
        const long long cc = min(c, n_chunks - 1);
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
        {
            wraw[nb] = *(const u32x4*)(a.W + w_base[nb] + cc * 1024 + (size_t)w_off);
            const uint8_t* sp = tiled_scales + s_base[nb] + cc * (16 * NS) + (size_t)s_off;
            if constexpr (NS == 8) { sraw[nb] = *(const u32x2*)sp; }
            else { sraw[nb] = u32x2{ *(const uint32_t*)sp, 0u }; }
        }
    };
    auto stage = [&](int buf) {
        u32x2* dst = (u32x2*)xs[buf];
#pragma unroll
        for (int i = 0; i < X_PER_THREAD; i++)
        {
            dst[x_store + i * (32 * CPR * 2)] = u32x2{ xreg[i][0], xreg[i][1] };
            dst[(x_store ^ 2) + i * (32 * CPR * 2)] = u32x2{ xreg[i][2], xreg[i][3] };
        }
    };
    // Half `half` (four elements, one scale block when BLOCK is 16) of dword d of the chunk, block nb -> two registers
    // of the lane's matrix-core operand: 2 conversions to FP32, 4 multiplies by the block scale, 2 packs to BF16
    auto dequant_half = [&](const u32x4* wraw, const u32x2* sraw, int nb, int d, int half, u32x4* wf) {
        const int si = BLOCK == 16 ? 2 * d + half : d;               // scale byte of the chunk
        const uint32_t sw = sraw[nb][si >> 2];
        const float sc = (si & 3) == 0 ? __builtin_amdgcn_cvt_f32_fp8(sw, 0) : (si & 3) == 1 ? __builtin_amdgcn_cvt_f32_fp8(sw, 1)
                       : (si & 3) == 2 ? __builtin_amdgcn_cvt_f32_fp8(sw, 2) : __builtin_amdgcn_cvt_f32_fp8(sw, 3);
        const uint32_t w = wraw[nb][d];
        const f32x2 v0 = half == 0 ? __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 0) : __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 2);
        const f32x2 v1 = half == 0 ? __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 1) : __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 3);
        const bf16x2 p0 = { (__bf16)(v0.x * sc), (__bf16)(v0.y * sc) };
        const bf16x2 p1 = { (__bf16)(v1.x * sc), (__bf16)(v1.y * sc) };
        wf[nb][2 * half] = __builtin_bit_cast(uint32_t, p0);
        wf[nb][2 * half + 1] = __builtin_bit_cast(uint32_t, p1);
    };

    // One 64-element half (h) of a chunk = two matrix-core steps of MB token blocks each.  The conversion of a step's
    // weights runs one step ahead of its products, a piece (half a dword: 9 VALU instructions) at a time between the
    // matrix-core instructions of one token block, so that neither pipe waits for the other: wf_a holds the operands of
    // the half's first step on entry and is refilled, during the second step, for the next half's first step; wf_b is
    // filled during the first step for the second.  Order: barrier | (first half: request the next chunk's codes and
    // scales) | first step | store the next activation tile to LDS, request the one after | second step; activation
    // fragments are read AHEAD token blocks in front of their use.  Scheduling fences keep that order.
    constexpr int AHEAD = 2;
    u32x4 wf_a[NB], wf_b[NB];
    auto k_tile = [&](int kt, int h, const u32x4* wcur, const u32x2* scur, u32x4* wnext, u32x2* snext) {
        __syncthreads();                                     // tile kt is in xs[kt & 1]; the other buffer is free
        if constexpr (MEM_BURSTS) { if (h == 0) { fetch_w(kt / 2 + 1, wnext, snext); } }
        const u32x4* xt = xs[kt & 1];
        constexpr int FRAGS = 2 * MB;
        static_assert(NB <= FRAGS && FRAGS / 2 + 1 + X_PER_THREAD <= FRAGS, "one token block per memory instruction");
        const long long w_cc = min(kt / 2 + 1, n_chunks - 1);
        const int x_k0 = min(kt + 2, n_kt - 1) * BK;
        constexpr int PIECES = 2 * NB;                       // per step
        auto read_frag = [&](int f) {
            const int row = (f % MB) * 16 + i16;
            return xt[row * CPR + swizzled_chunk_n<CPR>(row, 4 * (f / MB) + g)];
        };
        u32x4 ring[AHEAD + 1];
#pragma unroll
        for (int f = 0; f < AHEAD; f++) { ring[f] = read_frag(f); }
#pragma unroll
        for (int f = 0; f < FRAGS; f++)
        {
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (MEM_BURSTS)
            {
                if (f == FRAGS / 2)
                {
                    stage((kt + 1) & 1);
                    fetch_x(kt + 2);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            else
            {
                // one memory instruction (pair) per token block, as in the FP8 kernel: the next chunk's codes and scales
                // with the first blocks of a chunk's first half, the stores of the next activation tile from the middle
                // on, each followed one block later by the load that refills its register
                if (h == 0 && f < NB)
                {
                    wnext[f] = *(const u32x4*)(a.W + w_base[f] + w_cc * 1024 + (size_t)w_off);
                    const uint8_t* sp = tiled_scales + s_base[f] + w_cc * (16 * NS) + (size_t)s_off;
                    if constexpr (NS == 8) { snext[f] = *(const u32x2*)sp; }
                    else { snext[f] = u32x2{ *(const uint32_t*)sp, 0u }; }
                }
                if (f >= FRAGS / 2 && f < FRAGS / 2 + X_PER_THREAD)
                {
                    const int i = f - FRAGS / 2;
                    u32x2* dst = (u32x2*)xs[(kt + 1) & 1];
                    dst[x_store + i * (32 * CPR * 2)] = u32x2{ xreg[i][0], xreg[i][1] };
                    dst[(x_store ^ 2) + i * (32 * CPR * 2)] = u32x2{ xreg[i][2], xreg[i][3] };
                }
                if (f >= FRAGS / 2 + 1 && f < FRAGS / 2 + 1 + X_PER_THREAD)
                {
                    const int i = f - FRAGS / 2 - 1;
                    xreg[i] = *(const u32x4*)(x_begin + (size_t)x_k0 * 2 + (size_t)x_off[i]);
                }
            }
            if (f + AHEAD < FRAGS) { ring[(f + AHEAD) % (AHEAD + 1)] = read_frag(f + AHEAD); }
            const bf16x8 xf = __builtin_bit_cast(bf16x8, ring[f % (AHEAD + 1)]);
            const int st = f / MB, mb = f % MB;
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
            {
                const bf16x8 w = __builtin_bit_cast(bf16x8, st == 0 ? wf_a[nb] : wf_b[nb]);
                acc[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w, xf, acc[mb][nb], 0, 0, 0);
            }
            // this token block's share of the next step's conversions
            const int p_begin = mb * PIECES / MB, p_end = (mb + 1) * PIECES / MB;
#pragma unroll
            for (int p = p_begin; p < p_end; p++)
            {
                if (st == 0) { dequant_half(wcur, scur, p / 2, 2 * h + 1, p % 2, wf_b); }
                else if (h == 0) { dequant_half(wcur, scur, p / 2, 2, p % 2, wf_a); }
                else { dequant_half(wnext, snext, p / 2, 0, p % 2, wf_a); }
            }
            // one fragment read, then each matrix-core instruction followed by its share of the VALU work
            if (f + AHEAD < FRAGS) { __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); }
            constexpr int VALU_PER_MFMA = (9 * ((PIECES + MB - 1) / MB) + NB - 1) / NB;
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
            {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, VALU_PER_MFMA, 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    };

    fetch_x(0);
    fetch_w(0, wraw_a, sraw_a);
    stage(0);
    fetch_x(1);
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
    {
        dequant_half(wraw_a, sraw_a, nb, 0, 0, wf_a);
        dequant_half(wraw_a, sraw_a, nb, 0, 1, wf_a);
    }
    for (int c = 0; c < n_chunks; c += 2)
    {
        k_tile(2 * c, 0, wraw_a, sraw_a, wraw_b, sraw_b);
        k_tile(2 * c + 1, 1, wraw_a, sraw_a, wraw_b, sraw_b);
        if (c + 1 < n_chunks)
        {
            k_tile(2 * c + 2, 0, wraw_b, sraw_b, wraw_a, sraw_a);
            k_tile(2 * c + 3, 1, wraw_b, sraw_b, wraw_a, sraw_a);
        }
    }

    const bool wide_store = SPLIT ? a.n_out % 4 == 0 : (a.y_stride_out == 1 && a.y_stride_tok % 4 == 0 && ((uintptr_t)a.Y & 7u) == 0);
    if constexpr (PAIR && !SPLIT)
    {
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
        {
            const int tok = tok_base + mb * 16 + i16;
            if (tok >= a.tokens) { continue; }
#pragma unroll
            for (int nb = 0; nb < NBO; nb++)
            {
                const int out = out_base + nb * 16 + 4 * g;
                if (out >= a.n_out) { continue; }
                uint16_t o[4];
#pragma unroll
                for (int v = 0; v < 4; v++)
                {
                    const float gate = bf16_bits_to_f32(f32_to_bf16_bits(acc[mb][nb][v])), up = bf16_bits_to_f32(f32_to_bf16_bits(acc[mb][nb + NBO][v]));
                    const float sig = bf16_bits_to_f32(f32_to_bf16_bits(1.0f / (1.0f + expf(-gate))));
                    o[v] = (uint16_t)f32_to_bf16_bits(bf16_bits_to_f32(f32_to_bf16_bits(gate * sig)) * up);
                }
                uint16_t* y = a.Y + (long long)tok * a.y_stride_tok + (long long)out * a.y_stride_out;
                if (wide_store && out + 3 < a.n_out) { *(uint2*)y = uint2{ (uint32_t)o[0] | ((uint32_t)o[1] << 16), (uint32_t)o[2] | ((uint32_t)o[3] << 16) }; }
                else
                {
#pragma unroll
                    for (int v = 0; v < 4; v++)
                    {
                        if (out + v < a.n_out) { y[v * a.y_stride_out] = o[v]; }
                    }
                }
            }
        }
        return;
    }
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
    {
        const int tok = tok_base + mb * 16 + i16;
        if (tok >= a.tokens) { continue; }
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
        {
            const int out = out_base + (nb % NBO) * 16 + 4 * g;
            if (out >= a.n_out) { continue; }
            const f32x4 r = acc[mb][nb];
            if constexpr (SPLIT)
            {
                // pair: the up weight's sums are a second set behind all of the gate weight's
                float* p = partial + (((long long)(nb / NBO) * gridDim.y + blockIdx.y) * a.tokens + tok) * a.n_out + out;
                if (wide_store && out + 3 < a.n_out) { *(f32x4*)p = r; }
                else
                {
#pragma unroll
                    for (int v = 0; v < 4; v++)
                    {
                        if (out + v < a.n_out) { p[v] = r[v]; }
                    }
                }
            }
            else
            {
                uint16_t* y = a.Y + (long long)tok * a.y_stride_tok + (long long)out * a.y_stride_out;
                if (wide_store && out + 3 < a.n_out)
                {
                    uint16_t old[4] = { 0, 0, 0, 0 };
                    if (a.beta != 0.0f) { *(uint2*)old = *(const uint2*)y; }
                    uint16_t o[4];
#pragma unroll
                    for (int v = 0; v < 4; v++) { o[v] = finish_output_act<DT_BF16>(r[v], a.alpha, a.beta, &old[v]); }
                    *(uint2*)y = uint2{ (uint32_t)o[0] | ((uint32_t)o[1] << 16), (uint32_t)o[2] | ((uint32_t)o[3] << 16) };
                }
                else
                {
#pragma unroll
                    for (int v = 0; v < 4; v++)
                    {
                        if (out + v < a.n_out) { y[v * a.y_stride_out] = finish_output_act<DT_BF16>(r[v], a.alpha, a.beta, y + v * a.y_stride_out); }
                    }
                }
            }
        }
    }
}

// The combine launch of a k-split GEMM that also does what follows the linear in a transformer block: o = bf16(sum of the
// partial tiles), r = bf16(res + o), y = rmsnorm(r) * w -- gemm_splitk_combine_kernel, the residual add and the row norm
// in one launch, with their roundings and their order of sums (the sum of squares runs as in rms_norm_rows_kernel: lane l of
// one wave adds the 8-value chunks l, l + 64, ... in turn, then the wave reduction), so the bits are those of the three
// launches.  One 512-thread workgroup per token row, a thread per chunk of 8 features (n_out <= 4096, a multiple of 8);
// the loads of up to MAXS partial tiles are all issued before the first add.
template <int MAXS>
__global__ __launch_bounds__(512) void gemm_splitk_combine_add_norm_kernel(const float* __restrict__ partial, const int splits, const LinearArgs a, const AddNormArgs e)
{
    __shared__ float sq[512];
    __shared__ float s_invstd;
    const int row = blockIdx.x, c = threadIdx.x;
    const int n_chunks = a.n_out / 8;
    const bool active = c < n_chunks;
    const long long slice = (long long)a.tokens * a.n_out;
    const size_t at = (size_t)row * a.n_out + (size_t)min(c, n_chunks - 1) * 8;
    f32x4 lo[MAXS], hi[MAXS];
#pragma unroll
    for (int s = 0; s < MAXS; s++)
    {
        const float* p = partial + (long long)min(s, splits - 1) * slice + at;       // ranges past the last re-read it and are dropped
        lo[s] = *(const f32x4*)p;
        hi[s] = *(const f32x4*)(p + 4);
    }
    const u32x4 res = *(const u32x4*)(e.res + at), w = *(const u32x4*)(e.norm_w + (size_t)min(c, n_chunks - 1) * 8);
    f32x4 r0 = lo[0], r1 = hi[0];
#pragma unroll
    for (int s = 1; s < MAXS; s++)
    {
        if (s < splits)
        {
            r0 += lo[s];
            r1 += hi[s];
        }
    }
    u32x4 v;
#pragma unroll
    for (int d = 0; d < 4; d++)
    {
        const float o_lo = d < 2 ? r0[2 * d] : r1[2 * d - 4], o_hi = d < 2 ? r0[2 * d + 1] : r1[2 * d - 3];
        const float x_lo = bf16_bits_to_f32(res[d] & 0xFFFFu) + bf16_bits_to_f32(finish_output_act<DT_BF16>(o_lo, a.alpha, 0.0f, nullptr));
        const float x_hi = bf16_bits_to_f32(res[d] >> 16) + bf16_bits_to_f32(finish_output_act<DT_BF16>(o_hi, a.alpha, 0.0f, nullptr));
        v[d] = f32_to_bf16_bits(x_lo) | (f32_to_bf16_bits(x_hi) << 16);
    }
    if (active) { *(u32x4*)(e.sum + at) = v; }
    sq[c] = active ? sumsq8(v) : 0.0f;
    __syncthreads();
    if (c < 64)
    {
        float sumsq = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; j++) { sumsq += sq[c + 64 * j]; }
        const float invstd = rsqrtf(wave_sum(sumsq) / (float)a.n_out + e.eps);
        if (c == 0) { s_invstd = invstd; }
    }
    __syncthreads();
    if (active) { *(u32x4*)(e.y + at) = normed8(v, w, s_invstd); }
}

// the combine launch of a k-split GEMM: plain, or with the residual add and the norm behind the linear
template <int AT>
inline void launch_splitk_combine(const float* partial, int splits, const LinearArgs& a, const AddNormArgs* e)
{
    if (e)
    {
        if (splits <= 4) { gemm_splitk_combine_add_norm_kernel<4><<<a.tokens, 512, 0, stream()>>>(partial, splits, a, *e); }
        else if (splits <= 8) { gemm_splitk_combine_add_norm_kernel<8><<<a.tokens, 512, 0, stream()>>>(partial, splits, a, *e); }
        else { gemm_splitk_combine_add_norm_kernel<16><<<a.tokens, 512, 0, stream()>>>(partial, splits, a, *e); }
        return;
    }
    const long long groups = (long long)a.tokens * (a.n_out / 4);
    const long long blocks = (groups + 255) / 256;
    const long long cap = (long long)cu_count() * 16;
    gemm_splitk_combine_kernel<AT><<<(unsigned)(blocks < cap ? blocks : cap), 256, 0, stream()>>>(partial, splits, a);
}

// a.W = the tiled codes; splits > 1: `partial` holds splits * tokens * n_out floats
template <int BLOCK, int MB, int NB = 4>
void launch_gemm4_mfma_direct(const LinearArgs& a, const uint8_t* tiled_scales, int splits = 1, float* partial = nullptr, const AddNormArgs* e = nullptr)
{
    const int n_tiles = (a.n_out + 64 * NB - 1) / (64 * NB);
    const int m_tiles = (a.tokens + MB * 16 - 1) / (MB * 16);
    const dim3 grid(((n_tiles + 7) & ~7) * m_tiles, splits);
    if (splits > 1)
    {
        gemm4_mfma_direct_kernel<BLOCK, MB, true, NB><<<grid, 256, 0, stream()>>>(a, tiled_scales, n_tiles, partial);
        launch_splitk_combine<DT_BF16>(partial, splits, a, e);
    }
    else { gemm4_mfma_direct_kernel<BLOCK, MB, false, NB><<<grid, 256, 0, stream()>>>(a, tiled_scales, n_tiles, nullptr); }
}

// splits > 1: `partial` holds splits * tokens * n_out floats
template <int WT, int MB, bool TILED, int AT = DT_BF16, int NB = 4>
void launch_gemm_mfma_direct(const LinearArgs& a, int splits = 1, float* partial = nullptr, const AddNormArgs* e = nullptr)
{
    const int n_tiles = (a.n_out + 64 * NB - 1) / (64 * NB);
    const int m_tiles = (a.tokens + MB * 16 - 1) / (MB * 16);
    const dim3 grid(((n_tiles + 7) & ~7) * m_tiles, splits);
    const bool scaled = a.w_scale != 1.0f;
    if (splits > 1)
    {
        constexpr int PD = MB <= 4 ? 3 : 1;          // 64- and 32-token tiles split k only up to 64 tokens: bound by the weight bytes
        if (scaled) { gemm_mfma_direct_kernel<WT, true, MB, true, TILED, AT, NB, false, false, PD><<<grid, 256, 0, stream()>>>(a, n_tiles, partial); }
        else { gemm_mfma_direct_kernel<WT, false, MB, true, TILED, AT, NB, false, false, PD><<<grid, 256, 0, stream()>>>(a, n_tiles, partial); }
        launch_splitk_combine<AT>(partial, splits, a, e);
    }
    else
    {
        if (scaled) { gemm_mfma_direct_kernel<WT, true, MB, false, TILED, AT, NB><<<grid, 256, 0, stream()>>>(a, n_tiles, nullptr); }
        else { gemm_mfma_direct_kernel<WT, false, MB, false, TILED, AT, NB><<<grid, 256, 0, stream()>>>(a, n_tiles, nullptr); }
    }
}

// FP4 (tiled copies, K % 128 == 0): 64-token x 256-feature tiles, two workgroups per CU
template <int BLOCK>
void launch_gemm4_mfma_direct_segments(LinearArgs a)
{
    int n_tiles = 0;
    for (int s = 0; s < 3; s++)
    {
        a.seg_tile0[s] = n_tiles;
        if (s < a.n_segments) { n_tiles += (a.seg_n_out[s] + 255) / 256; }
    }
    a.seg_tile0[3] = n_tiles;
    for (int s = a.n_segments; s < 3; s++) { a.seg_tile0[s] = n_tiles; }
    // few tiles: the k range split over workgroups and one combine launch for all segments, as for FP8 below
    {
        const int cus = cu_count();
        int n_all = 0;
        bool by4 = true;
        for (int sg = 0; sg < 3; sg++)
        {
            if (sg >= a.n_segments) { a.seg_n_out[sg] = 0; }
            n_all += a.seg_n_out[sg];
            by4 = by4 && a.seg_n_out[sg] % 4 == 0;
        }
        const int mb = a.tokens > 64 ? 8 : 4;
        const int m_tiles = (a.tokens + mb * 16 - 1) / (mb * 16);
        long long splits = cus / ((long long)n_tiles * m_tiles);
        if (splits > (mb == 8 ? 8 : 16)) { splits = mb == 8 ? 8 : 16; }
        if (splits > a.K / 512) { splits = a.K / 512; }
        float* partial = splits >= 2 && by4 ? (float*)workspace((size_t)splits * a.tokens * n_all * sizeof(float)) : nullptr;
        if (partial)
        {
            const dim3 grid(((n_tiles + 7) & ~7) * m_tiles, (unsigned)splits);
            if (mb == 8) { gemm4_mfma_direct_kernel<BLOCK, 8, true, 4, true><<<grid, 256, 0, stream()>>>(a, nullptr, n_tiles, partial); }
            else { gemm4_mfma_direct_kernel<BLOCK, 4, true, 4, true><<<grid, 256, 0, stream()>>>(a, nullptr, n_tiles, partial); }
            const long long blocks = ((long long)a.tokens * (n_all / 4) + 255) / 256, cap = (long long)cus * 16;
            gemm_splitk_combine_kernel<DT_BF16, true, false><<<(unsigned)(blocks < cap ? blocks : cap), 256, 0, stream()>>>(partial, (int)splits, a);
            return;
        }
    }
    const dim3 grid(((n_tiles + 7) & ~7) * ((a.tokens + 63) / 64));
    gemm4_mfma_direct_kernel<BLOCK, 4, false, 4, true><<<grid, 256, 0, stream()>>>(a, nullptr, n_tiles, nullptr);
}

// FP4 gate / up pair with the SwiGLU product (tiled copies; a.W / a.W_pair = the copies, codes then scale bytes): 64 tokens
// x 128 output features per workgroup, the k range split when those are too few for the GPU
template <int BLOCK>
void launch_gemm4_mfma_direct_pair(const LinearArgs& a)
{
    const uint8_t* tiled_scales = a.W + (long long)((a.n_out + 15) / 16) * (a.K / 128) * 1024;
    const int n_tiles = (a.n_out + 127) / 128;
    const int m_tiles = (a.tokens + 63) / 64;
    long long splits = cu_count() / ((long long)n_tiles * m_tiles);
    if (splits > 8) { splits = 8; }
    if (splits > a.K / 512) { splits = a.K / 512; }
    float* partial = splits >= 2 && a.n_out % 4 == 0 ? (float*)workspace((size_t)2 * splits * a.tokens * a.n_out * sizeof(float)) : nullptr;
    if (partial)
    {
        const dim3 grid(((n_tiles + 7) & ~7) * m_tiles, (unsigned)splits);
        gemm4_mfma_direct_kernel<BLOCK, 4, true, 4, false, true><<<grid, 256, 0, stream()>>>(a, tiled_scales, n_tiles, partial);
        const long long blocks = ((long long)a.tokens * (a.n_out / 4) + 255) / 256, cap = (long long)cu_count() * 16;
        gemm_splitk_combine_kernel<DT_BF16, false, true><<<(unsigned)(blocks < cap ? blocks : cap), 256, 0, stream()>>>(partial, (int)splits, a);
        return;
    }
    const dim3 grid(((n_tiles + 7) & ~7) * m_tiles);
    gemm4_mfma_direct_kernel<BLOCK, 4, false, 4, false, true><<<grid, 256, 0, stream()>>>(a, tiled_scales, n_tiles, nullptr);
}

// up to three linears on the same activations in one launch: 64- or 128-token x 256-feature tiles, whichever gives the CUs
// two rounds of workgroups or more evenly
template <int WT, bool TILED>
void launch_gemm_mfma_direct_segments(LinearArgs a)
{
    const int cus = cu_count();
    int n_tiles = 0;
    for (int s = 0; s < 3; s++)
    {
        a.seg_tile0[s] = n_tiles;
        if (s < a.n_segments) { n_tiles += (a.seg_n_out[s] + 255) / 256; }
    }
    a.seg_tile0[3] = n_tiles;
    for (int s = a.n_segments; s < 3; s++) { a.seg_tile0[s] = n_tiles; }       // empty segments start past the last tile
    bool scaled = false;
    for (int s = 0; s < a.n_segments; s++) { scaled = scaled || a.seg_w_scale[s] != 1.0f; }
    const long long tiles8 = (long long)n_tiles * ((a.tokens + 127) / 128);
    const int n_pad = (n_tiles + 7) & ~7;
    // Few tiles (q, k, v of a 4096-wide model are 24 feature tiles; up to 512 tokens that is under one workgroup for every
    // second CU): the k range is split over workgroups as in plan_direct, every segment's partial sums laid out as its own
    // split GEMM one after the other, and one combine launch finishes all of them (36-layer model, 128 tokens: 8.0 -> 7.0 ms;
    // 256 tokens 8.4 -> 7.6; 512 tokens 10.8 -> 10.5).
    {
        int n_all = 0;
        bool by4 = true;
        for (int sg = 0; sg < 3; sg++)
        {
            if (sg >= a.n_segments) { a.seg_n_out[sg] = 0; }
            n_all += a.seg_n_out[sg];
            by4 = by4 && a.seg_n_out[sg] % 4 == 0;
        }
        const int mb = a.tokens > 64 ? 8 : (a.tokens > 32 ? 4 : 2);
        const long long base = (long long)n_tiles * ((a.tokens + mb * 16 - 1) / (mb * 16));
        long long splits = cus / base;
        if (splits > (mb == 8 ? 8 : 16)) { splits = mb == 8 ? 8 : 16; }
        if (splits > a.K / 512) { splits = a.K / 512; }
        float* partial = splits >= 2 && by4 ? (float*)workspace((size_t)splits * a.tokens * n_all * sizeof(float)) : nullptr;
        if (partial)
        {
            const dim3 grid(n_pad * ((a.tokens + mb * 16 - 1) / (mb * 16)), (unsigned)splits);
            if (mb == 8)
            {
                if (scaled) { gemm_mfma_direct_kernel<WT, true, 8, true, TILED, DT_BF16, 4, false, true><<<grid, 256, 0, stream()>>>(a, n_tiles, partial); }
                else { gemm_mfma_direct_kernel<WT, false, 8, true, TILED, DT_BF16, 4, false, true><<<grid, 256, 0, stream()>>>(a, n_tiles, partial); }
            }
            else if (mb == 4)
            {
                if (scaled) { gemm_mfma_direct_kernel<WT, true, 4, true, TILED, DT_BF16, 4, false, true, 3><<<grid, 256, 0, stream()>>>(a, n_tiles, partial); }
                else { gemm_mfma_direct_kernel<WT, false, 4, true, TILED, DT_BF16, 4, false, true, 3><<<grid, 256, 0, stream()>>>(a, n_tiles, partial); }
            }
            else
            {
                if (scaled) { gemm_mfma_direct_kernel<WT, true, 2, true, TILED, DT_BF16, 4, false, true, 3><<<grid, 256, 0, stream()>>>(a, n_tiles, partial); }
                else { gemm_mfma_direct_kernel<WT, false, 2, true, TILED, DT_BF16, 4, false, true, 3><<<grid, 256, 0, stream()>>>(a, n_tiles, partial); }
            }
            const long long blocks = ((long long)a.tokens * (n_all / 4) + 255) / 256, cap = (long long)cus * 16;
            gemm_splitk_combine_kernel<DT_BF16, true, false><<<(unsigned)(blocks < cap ? blocks : cap), 256, 0, stream()>>>(partial, (int)splits, a);
            return;
        }
    }
    // (on the file layout the 128-token tile is worth having from one workgroup per CU on, see plan_direct)
    if (a.tokens > 64 && (tiles8 >= 2LL * cus || (!TILED && tiles8 >= cus)))
    {
        const dim3 grid(n_pad * ((a.tokens + 127) / 128));
        if (scaled) { gemm_mfma_direct_kernel<WT, true, 8, false, TILED, DT_BF16, 4, false, true><<<grid, 256, 0, stream()>>>(a, n_tiles, nullptr); }
        else { gemm_mfma_direct_kernel<WT, false, 8, false, TILED, DT_BF16, 4, false, true><<<grid, 256, 0, stream()>>>(a, n_tiles, nullptr); }
    }
    else
    {
        const dim3 grid(n_pad * ((a.tokens + 63) / 64));
        if (scaled) { gemm_mfma_direct_kernel<WT, true, 4, false, TILED, DT_BF16, 4, false, true><<<grid, 256, 0, stream()>>>(a, n_tiles, nullptr); }
        else { gemm_mfma_direct_kernel<WT, false, 4, false, TILED, DT_BF16, 4, false, true><<<grid, 256, 0, stream()>>>(a, n_tiles, nullptr); }
    }
}

// gate / up pair with the SwiGLU product in the epilogue: 128 tokens x 128 output features per workgroup
template <int WT, bool TILED>
void launch_gemm_mfma_direct_pair(const LinearArgs& a)
{
    const int n_tiles = (a.n_out + 127) / 128;
    const int m_tiles = (a.tokens + 127) / 128;
    const bool scaled = a.w_scale != 1.0f || a.w_scale_pair != 1.0f;
    // Up to 128 tokens of a 12288-wide pair are 96 workgroups: the k range is split in two or more and the combine launch
    // adds the gate and the up sums and writes the SwiGLU product with the same roundings (36-layer model, 128 tokens:
    // 8.0 -> 7.3 ms; from 129 tokens on, 192 workgroups or more, the split only costs).
    {
        const int mb = a.tokens > 64 ? 8 : (a.tokens > 32 ? 4 : 2);
        const int m_split = (a.tokens + mb * 16 - 1) / (mb * 16);
        long long splits = cu_count() / ((long long)n_tiles * m_split);
        if (splits > 8) { splits = 8; }
        if (splits > a.K / 512) { splits = a.K / 512; }
        float* partial = splits >= 2 && a.n_out % 4 == 0 ? (float*)workspace((size_t)2 * splits * a.tokens * a.n_out * sizeof(float)) : nullptr;
        if (partial)
        {
            const dim3 grid(((n_tiles + 7) & ~7) * m_split, (unsigned)splits);
            if (mb == 8)
            {
                if (scaled) { gemm_mfma_direct_kernel<WT, true, 8, true, TILED, DT_BF16, 4, true><<<grid, 256, 0, stream()>>>(a, n_tiles, partial); }
                else { gemm_mfma_direct_kernel<WT, false, 8, true, TILED, DT_BF16, 4, true><<<grid, 256, 0, stream()>>>(a, n_tiles, partial); }
            }
            else if (mb == 4)
            {
                if (scaled) { gemm_mfma_direct_kernel<WT, true, 4, true, TILED, DT_BF16, 4, true, false, 3><<<grid, 256, 0, stream()>>>(a, n_tiles, partial); }
                else { gemm_mfma_direct_kernel<WT, false, 4, true, TILED, DT_BF16, 4, true, false, 3><<<grid, 256, 0, stream()>>>(a, n_tiles, partial); }
            }
            else
            {
                if (scaled) { gemm_mfma_direct_kernel<WT, true, 2, true, TILED, DT_BF16, 4, true, false, 3><<<grid, 256, 0, stream()>>>(a, n_tiles, partial); }
                else { gemm_mfma_direct_kernel<WT, false, 2, true, TILED, DT_BF16, 4, true, false, 3><<<grid, 256, 0, stream()>>>(a, n_tiles, partial); }
            }
            const long long blocks = ((long long)a.tokens * (a.n_out / 4) + 255) / 256, cap = (long long)cu_count() * 16;
            gemm_splitk_combine_kernel<DT_BF16, false, true><<<(unsigned)(blocks < cap ? blocks : cap), 256, 0, stream()>>>(partial, (int)splits, a);
            return;
        }
    }
    const dim3 grid(((n_tiles + 7) & ~7) * m_tiles);
    if (scaled) { gemm_mfma_direct_kernel<WT, true, 8, false, TILED, DT_BF16, 4, true><<<grid, 256, 0, stream()>>>(a, n_tiles, nullptr); }
    else { gemm_mfma_direct_kernel<WT, false, 8, false, TILED, DT_BF16, 4, true><<<grid, 256, 0, stream()>>>(a, n_tiles, nullptr); }
}

template <int WT, int BLOCK, int BM, int BN, int BK = 64, bool XCD = false, int AT = DT_BF16>
void launch_gemm_mfma(const LinearArgs& a)
{
    const int n_tiles = (a.n_out + BM - 1) / BM;
    const int m_tiles = (a.tokens + BN - 1) / BN;
    const int grid = XCD ? 8 * m_tiles * ((n_tiles + 7) / 8) : n_tiles * m_tiles;
    if (WT != DT_FP4 && a.w_scale != 1.0f) { gemm_mfma_kernel<WT, BLOCK, BM, BN, true, BK, XCD, AT><<<grid, 256, 0, stream()>>>(a, n_tiles, m_tiles); }
    else { gemm_mfma_kernel<WT, BLOCK, BM, BN, false, BK, XCD, AT><<<grid, 256, 0, stream()>>>(a, n_tiles, m_tiles); }
}

// Tile shape and k split of the register-fed kernels (tuned on MI355X with the FP8 kernel): a workgroup owns 64 NB features x
// 16 MB tokens.  A CU wants two resident workgroups (one alone reaches ~85 % of the rate), the workgroups should spread
// evenly over the CUs (384 tiles on 256 CUs leave half of them with twice the work: 36 % of peak where 512 even tiles
// reach 42 %), and 48-feature waves with 64-token tiles cost ~5 % against the larger tiles.  Too few tiles in every
// shape: the k range is split over workgroups (256-feature tiles, about one workgroup per CU, 1024 elements of k or more
// each; 512 or more up to 64 tokens) and a second kernel adds the partial sums.
struct DirectPlan
{
    int nb, mb, splits;
    float* partial;
    bool refused;            // a fixed scratch buffer is too small for the k split this shape takes (SplitScratch::refused says how much)
};

// Gives the plan `s` k ranges and the FP32 scratch they need; false when a fixed scratch buffer is too small for them.
inline bool attach_split(DirectPlan& plan, const LinearArgs& a, long long s, SplitScratch* scratch)
{
    if (s <= 1) { return true; }
    const size_t need = (size_t)s * a.tokens * a.n_out * sizeof(float);
    if (scratch && scratch->strict)
    {
        if (!scratch->fixed || need > scratch->fixed_bytes)
        {
            scratch->refused = need;
            plan.refused = true;
            return false;
        }
        plan.partial = scratch->fixed;
    }
    else { plan.partial = (float*)workspace(need); }
    if (plan.partial) { plan.splits = (int)s; }
    return true;
}

// fp4: the FP4 kernel's costs -- the 128-token x 256-feature tile stays out of the scoring (see plan_direct_fp4), and
// 64-token tiles pay for converting every weight for half as many products (913 against 1037 TFLOP/s at equal balance).
// row_major (FP8 only): the weight is read from the file layout, where a wave's load is sixteen half cache lines; 64-token
// tiles then pay that fetch for half as many products, and a 128-token tile is worth having even at one workgroup per CU
// (4096 x 4096 at 2048 tokens: 70 us against 91; K 12288: 196 against 244; on the tiled copy the two are level).
// 64 tokens x 128 features (FP8, K < 8192, at most 2048 features) puts 256 or more workgroups on outputs as narrow as 1024
// features (2048 tokens: 29 / 35 us tiled / row-major against 33 / 40).  Wider outputs with few tiles keep the k split: with
// a long K it is far ahead (K 12288 at 512 tokens: 60 against 110 us), and on 512 tokens x 4096 x 4096, where the two
// measure the same on weights that rotate through the memory-side cache, the split is 8 us ahead inside a whole model.
inline DirectPlan plan_direct(const LinearArgs& a, SplitScratch* scratch, bool fp4 = false, bool row_major = false)
{
    const int cus = cu_count();
    const bool big_tile = !fp4;
    struct Shape { int nb, mb; double quality; };
    const double q64 = row_major ? 0.8 : 1.0;            // what a 64-token tile is worth against a 128-token one
    const Shape shapes[] = { { 4, 8, 1.0 }, { 4, 4, fp4 ? 0.88 : q64 }, { 3, 8, 1.0 }, { 3, 4, fp4 ? 0.84 : 0.95 * q64 }, { 2, 4, 0.9 * q64 } };
    DirectPlan plan = { 4, 4, 1, nullptr, false };
    double best = -1.0;
    for (const Shape& sh : shapes)
    {
        if (sh.nb == 2 && (fp4 || a.K >= 8192 || a.n_out > 2048)) { continue; }
        if (sh.mb == 8 && (a.tokens <= 64 || (sh.nb == 4 && !big_tile))) { continue; }
        const long long tiles = (long long)((a.n_out + 64 * sh.nb - 1) / (64 * sh.nb)) * ((a.tokens + 16 * sh.mb - 1) / (16 * sh.mb));
        const double balance = (double)tiles / (double)(((tiles + cus - 1) / cus) * cus);
        double occupancy = tiles >= 2LL * cus ? 1.0 : (tiles > cus ? 0.95 : 0.85);
        // one 128 x 256 tile on (nearly) every CU and a long K: ahead of two 64-token tiles per CU, which convert every weight
        // twice (2048 tokens x 4096 features, K 12288, tiled copy: 160 against 168-170 us; K 4096: level)
        if (sh.nb == 4 && sh.mb == 8 && !row_major && a.K >= 8192 && tiles * 8 > 7LL * cus && tiles <= cus) { occupancy = 1.02; }
        const double score = sh.quality * balance * occupancy;
        if (score > best + 1e-9)
        {
            best = score;
            plan.nb = sh.nb;
            plan.mb = sh.mb;
        }
    }
    const long long n_tiles = (a.n_out + 255) / 256;
    const long long tiles8 = n_tiles * ((a.tokens + 127) / 128), tiles4 = n_tiles * ((a.tokens + 63) / 64);
    if (best < 0.6 && tiles4 * 4 < 5LL * cus && a.n_out % 4 == 0)
    {
        const long long base = a.tokens > 64 ? tiles8 : tiles4;
        long long s = (cus + base / 2) / base;
        // up to 64 tokens the weight bytes bound the launch and finer k ranges put more workgroups on them (32 tokens:
        // 4096 x 4096 17.3 -> 14.6 us, 1024 x 4096 16.3 -> 13.5, 4096 x 12288 28.5 -> 24.0); above that the FP32 partial
        // sums weigh more and a range keeps 1024 elements of k or more
        const long long s_max = a.tokens <= 64 ? 16 : 8, k_min = a.tokens <= 64 ? 512 : 1024;
        if (s > s_max) { s = s_max; }
        if (s > a.K / k_min) { s = a.K / k_min; }
        if (!attach_split(plan, a, s, scratch)) { return plan; }
        if (plan.splits > 1)
        {
            plan.nb = 4;
            plan.mb = a.tokens > 64 ? 8 : (a.tokens > 32 || fp4 ? 4 : 2);        // FP8, up to 32 tokens: a 32-token tile
        }
    }
    return plan;
}

// FP4: the 128 x 256 tile needs the register file of a whole SIMD per wave, so a CU runs one such workgroup at a time
// and nothing hides its prologue and epilogue: it pays when every tile gets a CU of its own (1009 TFLOP/s on
// 2048 x 4096, K 14336, against 940 for 64 x 256 tiles; 767 against 1009 for 128 x 192 tiles on 2048 x 14336, where a CU
// runs three or four of them in sequence), with the k range split when the tiles are few.
inline DirectPlan plan_direct_fp4(const LinearArgs& a, SplitScratch* scratch)
{
    const int cus = cu_count();
    const long long tiles = (long long)((a.n_out + 255) / 256) * ((a.tokens + 127) / 128);
    if (a.tokens > 64 && tiles <= cus)
    {
        long long s = a.n_out % 4 == 0 ? (cus + tiles / 2) / tiles : 1;
        if (s > 8) { s = 8; }
        if (s > a.K / 1024) { s = a.K / 1024; }
        if (s < 1) { s = 1; }
        if (tiles * s * 5 >= 3LL * cus)
        {
            DirectPlan plan = { 4, 8, 1, nullptr, false };
            attach_split(plan, a, s, scratch);
            return plan;
        }
    }
    return plan_direct(a, scratch, true);
}

// Kernel choice (tuned on MI355X).  FP8 weights with K a multiple of 64 and at least 17 tokens take the
// kernel that keeps the weights out of LDS -- on the tiled copy of the weight when one is registered
// (1.10-1.15x the row-major rate: a wave's load is then eight full cache lines instead of sixteen half
// lines).  The tile shape comes from plan_direct (128- or 64-token tiles of 256, 192 or 128 features, whichever spreads
// most evenly over the CUs); when none fills the machine the k range is split over workgroups (about one per CU, 16 k-tiles or more each) and a
// second kernel adds the partial sums -- 2x on 512 tokens x 4096 features x K 12288.  Everything else (FP4,
// ragged K) takes the two-operand kernel: 128 x 128 tiles with the XCD-aware order when they
// give every CU at least two workgroups (k step 128 for long K, where it halves the barriers per FLOP),
// otherwise 128 x 64 tiles to put more workgroups on the machine.
// `scratch`: see SplitScratch; nullptr = the stream's grow-on-demand workspace.  Returns false (nothing launched)
// only when a fixed scratch buffer is too small for the k-split this shape takes.
// `e`: the caller wants the residual add and the norm behind the linear in the combine launch of a k split; false
// (nothing launched) when this shape does not split.
template <int WT, int BLOCK, int AT = DT_BF16>
bool gemm_mfma(const LinearArgs& a, const uint8_t* tiled = nullptr, SplitScratch* scratch = nullptr, const AddNormArgs* e = nullptr)
{
    if constexpr (WT == DT_FP4 && AT == DT_BF16)
    {
        // FP4 with a tiled copy (codes, then the scales behind all code KiBs): the register-fed kernel
        if (tiled && a.K % 128 == 0 && a.tokens >= (e ? 2 : 17) && (long long)a.tokens * a.ldx * 2 < (1LL << 32))
        {
            LinearArgs d = a;
            d.W = tiled;
            const uint8_t* scales = tiled + (long long)((a.n_out + 15) / 16) * (a.K / 128) * 1024;
            const DirectPlan plan = plan_direct_fp4(a, scratch);
            if (plan.refused || (e && plan.splits <= 1)) { return false; }
            if (plan.nb == 3) { plan.mb == 8 ? launch_gemm4_mfma_direct<BLOCK, 8, 3>(d, scales) : launch_gemm4_mfma_direct<BLOCK, 4, 3>(d, scales); }
            else if (plan.mb == 8) { launch_gemm4_mfma_direct<BLOCK, 8>(d, scales, plan.splits, plan.partial, e); }
            else { launch_gemm4_mfma_direct<BLOCK, 4>(d, scales, plan.splits, plan.partial, e); }
            return true;
        }
    }
    if constexpr (AT != DT_BF16) { if (e) { return false; } }
    if constexpr (WT != DT_FP4)
    {
        const bool small_offsets = (long long)a.n_out * a.ldw < (1LL << 32) && (long long)a.tokens * a.ldx * 2 < (1LL << 32);
        // (HALF activations: the register-fed kernel also serves 5-16 tokens where the matrix-core GEMV refuses the shape)
        if (a.K % 64 == 0 && a.tokens >= (e ? 2 : (AT == DT_HALF ? 5 : 17)) && small_offsets)
        {
            LinearArgs d = a;
            if (tiled) { d.W = tiled; }
            const DirectPlan plan = plan_direct(a, scratch, false, tiled == nullptr);
            if (plan.refused || (e && plan.splits <= 1)) { return false; }
            const int nb = plan.nb, mb = plan.mb, splits = plan.splits;
            float* const partial = plan.partial;
            if (nb == 2) { tiled ? launch_gemm_mfma_direct<WT, 4, true, AT, 2>(d) : launch_gemm_mfma_direct<WT, 4, false, AT, 2>(d); }
            else if (tiled)
            {
                if (nb == 3) { mb == 8 ? launch_gemm_mfma_direct<WT, 8, true, AT, 3>(d) : launch_gemm_mfma_direct<WT, 4, true, AT, 3>(d); }
                else if (mb == 8) { launch_gemm_mfma_direct<WT, 8, true, AT>(d, splits, partial, e); }
                else if (mb == 2 && splits > 1) { launch_gemm_mfma_direct<WT, 2, true, AT>(d, splits, partial, e); }
                else { launch_gemm_mfma_direct<WT, 4, true, AT>(d, splits, partial, e); }
            }
            else
            {
                if (nb == 3) { mb == 8 ? launch_gemm_mfma_direct<WT, 8, false, AT, 3>(d) : launch_gemm_mfma_direct<WT, 4, false, AT, 3>(d); }
                else if (mb == 8) { launch_gemm_mfma_direct<WT, 8, false, AT>(d, splits, partial, e); }
                else if (mb == 2 && splits > 1) { launch_gemm_mfma_direct<WT, 2, false, AT>(d, splits, partial, e); }
                else { launch_gemm_mfma_direct<WT, 4, false, AT>(d, splits, partial, e); }
            }
            return true;
        }
    }
    if (e) { return false; }
    const long long tiles_big = (long long)((a.n_out + 127) / 128) * ((a.tokens + 127) / 128);
    if (tiles_big >= 2LL * cu_count())
    {
        if (a.K >= 8192) { launch_gemm_mfma<WT, BLOCK, 128, 128, 128, true, AT>(a); }
        else { launch_gemm_mfma<WT, BLOCK, 128, 128, 64, true, AT>(a); }
    }
    else { launch_gemm_mfma<WT, BLOCK, 128, 64, 64, false, AT>(a); }
    return true;
}

}    // namespace ccq
