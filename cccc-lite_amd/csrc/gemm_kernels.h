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

template <int WT, int BLOCK, int BM, int BN, int BK = 64, bool XCD = false, int AT = DT_BF16>
void launch_gemm_mfma(const LinearArgs& a)
{
    const int n_tiles = (a.n_out + BM - 1) / BM;
    const int m_tiles = (a.tokens + BN - 1) / BN;
    const int grid = XCD ? 8 * m_tiles * ((n_tiles + 7) / 8) : n_tiles * m_tiles;
    if (WT != DT_FP4 && a.w_scale != 1.0f) { gemm_mfma_kernel<WT, BLOCK, BM, BN, true, BK, XCD, AT><<<grid, 256, 0, stream()>>>(a, n_tiles, m_tiles); }
    else { gemm_mfma_kernel<WT, BLOCK, BM, BN, false, BK, XCD, AT><<<grid, 256, 0, stream()>>>(a, n_tiles, m_tiles); }
}

// Tile choice (tuned on MI355X): 128 x 128 tiles with the XCD-aware order when they give every CU at
// least two workgroups (k step 128 for long K, where it halves the barriers per FLOP), otherwise
// 128 x 64 tiles to put more workgroups on the machine.
template <int WT, int BLOCK, int AT = DT_BF16>
bool gemm_mfma(const LinearArgs& a)
{
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
