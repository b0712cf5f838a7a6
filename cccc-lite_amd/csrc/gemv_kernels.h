// Decode-time GEMV family for gfx950 (tokens 1..16): streams the packed weight once with 128-bit
// loads, converts FP8 / FP4 to BF16 in registers with the CDNA4 conversion instructions, multiplies
// against BF16 activations with FP32 accumulation and rounds once to BF16.
//
// Numerics are those of the reference's "dequantise to BF16, then BF16 GEMM with FP32 accumulate"
// (cccc/cublas_real.h:943-964): the weight value entering each product is bf16(decode(w) * scale).
//   * scale == 1: every E5M2 / E4M3 / E2M1 value is exactly representable in BF16, so the hardware
//     conversion is that value.
//   * scale != 1: decode to FP32, one FP32 multiply, round to nearest even to BF16 (SCALED = true).
//   * FP4 block scales: fp4 * e4m3 has at most 6 significant bits, so bf16(fp4 * s) == fp4 * s and
//     sum_k (fp4_k * s_b) * x_k == sum_b s_b * sum_{k in b} fp4_k * x_k; the kernel factors the
//     scale out of each block.
#pragma once
#include "linear_args.h"
#include "quant_device.h"

namespace ccq
{

// ------------------------------------------------------------------------------------------
// register-level conversions

// four FP8 codes in one dword -> two packed BF16 pairs (elements 0,1 and 2,3)
template <int WT, bool SCALED>
__device__ __forceinline__ void fp8x4_to_bf16(uint32_t w, float scale, bf16x2& p01, bf16x2& p23)
{
    if (!SCALED)
    {
        if (WT == DT_E5M2)
        {
            p01 = __builtin_amdgcn_cvt_scalef32_pk_bf16_bf8(w, 1.0f, false);
            p23 = __builtin_amdgcn_cvt_scalef32_pk_bf16_bf8(w, 1.0f, true);
        }
        else
        {
            p01 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, false);
            p23 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, true);
        }
    }
    else
    {
        f32x2 a, b;
        if (WT == DT_E5M2)
        {
            a = __builtin_amdgcn_cvt_pk_f32_bf8(w, false);
            b = __builtin_amdgcn_cvt_pk_f32_bf8(w, true);
        }
        else
        {
            a = __builtin_amdgcn_cvt_pk_f32_fp8(w, false);
            b = __builtin_amdgcn_cvt_pk_f32_fp8(w, true);
        }
        p01 = bf16x2{ (__bf16)(a.x * scale), (__bf16)(a.y * scale) };
        p23 = bf16x2{ (__bf16)(b.x * scale), (__bf16)(b.y * scale) };
    }
}

__device__ __forceinline__ float dot2_bf16(bf16x2 a, uint32_t x, float acc)
{
    return __builtin_amdgcn_fdot2_f32_bf16(a, __builtin_bit_cast(bf16x2, x), acc, false);
}

// The same two steps for either 16-bit activation type.  HALF: the weight entering a product is
// half(decode(w) * scale) (cccc/cublas_real.h:921-938); every E5M2 / E4M3 value is a half exactly.
template <int AT>
struct ActPair
{
    typedef bf16x2 type;
};
template <>
struct ActPair<DT_HALF>
{
    typedef f16x2 type;
};

template <int WT, bool SCALED, int AT>
__device__ __forceinline__ void fp8x4_to_pairs(uint32_t w, float scale, typename ActPair<AT>::type& p01, typename ActPair<AT>::type& p23)
{
    if constexpr (AT == DT_BF16) { fp8x4_to_bf16<WT, SCALED>(w, scale, p01, p23); }
    else if constexpr (!SCALED)
    {
        if (WT == DT_E5M2)
        {
            p01 = __builtin_amdgcn_cvt_scalef32_pk_f16_bf8(w, 1.0f, false);
            p23 = __builtin_amdgcn_cvt_scalef32_pk_f16_bf8(w, 1.0f, true);
        }
        else
        {
            p01 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, false);
            p23 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, true);
        }
    }
    else
    {
        f32x2 a, b;
        if (WT == DT_E5M2)
        {
            a = __builtin_amdgcn_cvt_pk_f32_bf8(w, false);
            b = __builtin_amdgcn_cvt_pk_f32_bf8(w, true);
        }
        else
        {
            a = __builtin_amdgcn_cvt_pk_f32_fp8(w, false);
            b = __builtin_amdgcn_cvt_pk_f32_fp8(w, true);
        }
        p01 = f16x2{ (_Float16)(a.x * scale), (_Float16)(a.y * scale) };
        p23 = f16x2{ (_Float16)(b.x * scale), (_Float16)(b.y * scale) };
    }
}

template <int AT>
__device__ __forceinline__ float dot2_act(typename ActPair<AT>::type a, uint32_t x, float acc)
{
    if constexpr (AT == DT_BF16) { return dot2_bf16(a, x, acc); }
    else { return __builtin_amdgcn_fdot2(a, __builtin_bit_cast(f16x2, x), acc, false); }
}

// ------------------------------------------------------------------------------------------
// Activations in LDS.  A "k-step" is the span one wave covers with one 128-bit load per lane:
// KSTEP elements.  Each lane needs KSTEP/64 consecutive BF16 of every token per step; they are
// stored as PARTS 16-byte pieces, piece p of lane l at [step][token][p][l], so that every
// ds_read_b128 of a wave hits 64 consecutive 16-byte slots (no bank conflicts).
//   FP8: KSTEP = 1024, PARTS = 2.   FP4: KSTEP = 2048, PARTS = 4.

template <int MT, int PARTS>
__device__ __forceinline__ void stage_activations(const LinearArgs& a, u32x4* xs, int n_steps, int threads)
{
    constexpr int KSTEP = 64 * 8 * PARTS;
    const int chunks_per_token = n_steps * 64 * PARTS;    // 16-byte chunks, zero padded beyond K
    for (int c = threadIdx.x; c < chunks_per_token * MT; c += threads)
    {
        const int t = c / chunks_per_token;
        const int r = c - t * chunks_per_token;    // chunk index along k
        const int k = r * 8;
        u32x4 v = { 0u, 0u, 0u, 0u };
        if (k < a.K) { v = *(const u32x4*)(a.X + (long long)t * a.ldx + k); }
        const int step = k / KSTEP;
        const int in_step = r - step * (64 * PARTS);
        const int lane = in_step / PARTS;
        const int part = in_step - lane * PARTS;
        xs[((step * MT + t) * PARTS + part) * 64 + lane] = v;
    }
}

// ------------------------------------------------------------------------------------------
// FP8 GEMV, dot2 + DPP reduction.  One wave owns R consecutive output rows; lanes stride along K.
//   WT      DT_E5M2 / DT_E4M3
//   MT      tokens handled (1..4), compile time so the accumulators stay in registers
//   R       rows per wave
//   U       k-steps in flight per loop trip (loads issued before any is consumed)
//   WAVES   waves per workgroup
// Requires: K % 16 == 0, ldw % 16 == 0, W 16-byte aligned, ldx % 8 == 0, X 16-byte aligned.
// Dynamic LDS: MT * ceil(K / 1024) * 2048 bytes.

template <int WT, int MT, int R, int U, int WAVES, bool SCALED, int AT = DT_BF16>
__global__ __launch_bounds__(WAVES * 64) void gemv8_dot2_kernel(const LinearArgs a)
{
    extern __shared__ u32x4 xs[];
    const int n_steps = (a.K + 1023) / 1024;
    stage_activations<MT, 2>(a, xs, n_steps, WAVES * 64);
    __syncthreads();

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n_groups = (a.n_out + R - 1) / R;
    const int last_row = a.n_out - 1;

    for (int g = blockIdx.x * WAVES + wave; g < n_groups; g += gridDim.x * WAVES)
    {
        const uint8_t* wrow[R];
#pragma unroll
        for (int r = 0; r < R; r++)
        {
            const int row = min(g * R + r, last_row);    // clamped rows are computed and dropped
            wrow[r] = a.W + (long long)row * a.ldw + lane * 16;
        }
        float acc[R][MT];
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int t = 0; t < MT; t++) { acc[r][t] = 0.0f; }

        for (int s0 = 0; s0 < n_steps; s0 += U)
        {
            u32x4 w[U][R];
#pragma unroll
            for (int u = 0; u < U; u++)
            {
                const int k = (s0 + u) * 1024 + lane * 16;
#pragma unroll
                for (int r = 0; r < R; r++)
                {
                    w[u][r] = u32x4{ 0u, 0u, 0u, 0u };
                    if (k < a.K) { w[u][r] = __builtin_nontemporal_load((const u32x4*)(wrow[r] + (s0 + u) * 1024)); }
                }
            }
#pragma unroll
            for (int u = 0; u < U; u++)
            {
                if (s0 + u < n_steps)
                {
                    u32x4 x[MT][2];
#pragma unroll
                    for (int t = 0; t < MT; t++)
                    {
                        x[t][0] = xs[(((s0 + u) * MT + t) * 2 + 0) * 64 + lane];
                        x[t][1] = xs[(((s0 + u) * MT + t) * 2 + 1) * 64 + lane];
                    }
#pragma unroll
                    for (int r = 0; r < R; r++)
                    {
#pragma unroll
                        for (int d = 0; d < 4; d++)
                        {
                            typename ActPair<AT>::type p01, p23;
                            fp8x4_to_pairs<WT, SCALED, AT>(w[u][r][d], a.w_scale, p01, p23);
#pragma unroll
                            for (int t = 0; t < MT; t++)
                            {
                                acc[r][t] = dot2_act<AT>(p01, x[t][d >> 1][(d & 1) * 2 + 0], acc[r][t]);
                                acc[r][t] = dot2_act<AT>(p23, x[t][d >> 1][(d & 1) * 2 + 1], acc[r][t]);
                            }
                        }
                    }
                }
            }
        }

#pragma unroll
        for (int r = 0; r < R; r++)
        {
#pragma unroll
            for (int t = 0; t < MT; t++)
            {
                const float total = wave_sum(acc[r][t]);
                const int row = g * R + r;
                if (lane == 0 && row < a.n_out)
                {
                    uint16_t* y = a.Y + (long long)t * a.y_stride_tok + (long long)row * a.y_stride_out;
                    *y = finish_output_act<AT>(total, a.alpha, a.beta, y);
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// FP8 GEMV, dot2 + DPP reduction, software pipelined.  Same decomposition as gemv8_dot2_kernel, but
// the (row group, k trip) pairs a wave walks are flattened into one sequence and the 128-bit loads
// of the next pair are issued before the current pair is multiplied, so every wave always has
// U * R KiB in flight -- including across the activation staging barrier at kernel start.
//   NT      non-temporal weight loads

template <bool NT>
__device__ __forceinline__ u32x4 load_w128(const uint8_t* p)
{
    return NT ? __builtin_nontemporal_load((const u32x4*)p) : *(const u32x4*)p;
}

template <int WT, int MT, int R, int U, int WAVES, bool SCALED, bool NT>
__global__ __launch_bounds__(WAVES * 64) void gemv8_dot2_pipe_kernel(const LinearArgs a)
{
    extern __shared__ u32x4 xs[];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n_steps = (a.K + 1023) / 1024;
    const int trips = (n_steps + U - 1) / U;
    const int n_groups = (a.n_out + R - 1) / R;
    const int last_row = a.n_out - 1;
    const int g0 = blockIdx.x * WAVES + wave;
    const int g_stride = gridDim.x * WAVES;
    const int my_groups = g0 < n_groups ? (n_groups - g0 + g_stride - 1) / g_stride : 0;
    const int total = my_groups * trips;

    auto issue = [&](int it, u32x4 (&w)[U][R]) {
        const int gi = it / trips;
        const int s0 = (it - gi * trips) * U;
        const int g = g0 + gi * g_stride;
#pragma unroll
        for (int r = 0; r < R; r++)
        {
            const int row = min(g * R + r, last_row);
            const uint8_t* base = a.W + (long long)row * a.ldw + lane * 16;
#pragma unroll
            for (int u = 0; u < U; u++)
            {
                const int k = (s0 + u) * 1024 + lane * 16;
                w[u][r] = u32x4{ 0u, 0u, 0u, 0u };
                if (k < a.K) { w[u][r] = load_w128<NT>(base + (s0 + u) * 1024); }
            }
        }
    };

    float acc[R][MT];
    auto compute = [&](int it, const u32x4 (&w)[U][R]) {
        const int gi = it / trips;
        const int trip = it - gi * trips;
        const int s0 = trip * U;
        if (trip == 0)
        {
#pragma unroll
            for (int r = 0; r < R; r++)
#pragma unroll
                for (int t = 0; t < MT; t++) { acc[r][t] = 0.0f; }
        }
#pragma unroll
        for (int u = 0; u < U; u++)
        {
            if (s0 + u < n_steps)
            {
                u32x4 x[MT][2];
#pragma unroll
                for (int t = 0; t < MT; t++)
                {
                    x[t][0] = xs[(((s0 + u) * MT + t) * 2 + 0) * 64 + lane];
                    x[t][1] = xs[(((s0 + u) * MT + t) * 2 + 1) * 64 + lane];
                }
#pragma unroll
                for (int r = 0; r < R; r++)
                {
#pragma unroll
                    for (int d = 0; d < 4; d++)
                    {
                        bf16x2 p01, p23;
                        fp8x4_to_bf16<WT, SCALED>(w[u][r][d], a.w_scale, p01, p23);
#pragma unroll
                        for (int t = 0; t < MT; t++)
                        {
                            acc[r][t] = dot2_bf16(p01, x[t][d >> 1][(d & 1) * 2 + 0], acc[r][t]);
                            acc[r][t] = dot2_bf16(p23, x[t][d >> 1][(d & 1) * 2 + 1], acc[r][t]);
                        }
                    }
                }
            }
        }
        if (trip == trips - 1)
        {
            const int g = g0 + gi * g_stride;
#pragma unroll
            for (int r = 0; r < R; r++)
            {
#pragma unroll
                for (int t = 0; t < MT; t++)
                {
                    const float sum = wave_sum(acc[r][t]);
                    const int row = g * R + r;
                    if (lane == 0 && row < a.n_out)
                    {
                        uint16_t* y = a.Y + (long long)t * a.y_stride_tok + (long long)row * a.y_stride_out;
                        *y = finish_output(sum, a.alpha, a.beta, y);
                    }
                }
            }
        }
    };

    u32x4 wa[U][R], wb[U][R];
    if (total > 0) { issue(0, wa); }
    stage_activations<MT, 2>(a, xs, n_steps, WAVES * 64);
    __syncthreads();
    for (int it = 0; it < total; it += 2)
    {
        if (it + 1 < total) { issue(it + 1, wb); }
        compute(it, wa);
        if (it + 2 < total) { issue(it + 2, wa); }
        if (it + 1 < total) { compute(it + 1, wb); }
    }
}

// ------------------------------------------------------------------------------------------
// FP4 block-scale GEMV, dot2 + DPP reduction.  One 128-bit load = 32 nibbles = 32 consecutive
// elements of one row = 32 / BLOCK blocks (BLOCK = 16 or 32); the block scales of a k-step are
// 64 * 32 / BLOCK consecutive bytes of the scale array.
// Requires: K % 32 == 0, ldw == K (blocks run over the flat index), W 16-byte aligned,
// (row * K) % BLOCK == 0, ldx % 8 == 0, X 16-byte aligned.
// Dynamic LDS: MT * ceil(K / 2048) * 4096 bytes.

__device__ __forceinline__ float e4m3_byte_to_f32(uint32_t word, int byte_index)
{
    return byte_index == 0 ? __builtin_amdgcn_cvt_f32_fp8(word, 0) : __builtin_amdgcn_cvt_f32_fp8(word, 1);
}

// RAGGED (BLOCK 16 only): K % 32 == 16, legal in the reference, whose blocks of 16 run over the flat element index
// (cccc-cuda/cuda_functions.cu:2926-2939).  Every other row then starts 8 bytes off a 16-byte boundary and at an odd
// scale byte, and a row's last load covers 16 elements of this row and 16 of the next: codes are fetched as two 8-byte
// halves and scales as single bytes, and the half that belongs to the next row is neither read nor used.
template <int MT, int R, int U, int WAVES, int BLOCK, bool RAGGED = false>
__global__ __launch_bounds__(WAVES * 64) void gemv4_dot2_kernel(const LinearArgs a)
{
    static_assert(BLOCK == 16 || BLOCK == 32, "block scale length");
    static_assert(!RAGGED || BLOCK == 16, "ragged rows: blocks of 16 only (blocks of 32 would straddle rows)");
    extern __shared__ u32x4 xs[];
    const int n_steps = (a.K + 2047) / 2048;
    stage_activations<MT, 4>(a, xs, n_steps, WAVES * 64);
    __syncthreads();

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n_groups = (a.n_out + R - 1) / R;
    const int last_row = a.n_out - 1;

    for (int g = blockIdx.x * WAVES + wave; g < n_groups; g += gridDim.x * WAVES)
    {
        const uint8_t* wrow[R];
        const uint8_t* srow[R];
#pragma unroll
        for (int r = 0; r < R; r++)
        {
            const long long row = min(g * R + r, last_row);
            wrow[r] = a.W + ((row * a.ldw) >> 1) + lane * 16;
            srow[r] = a.blk_sc + (row * a.ldw) / BLOCK + lane * (32 / BLOCK);
        }
        float acc[R][MT];
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int t = 0; t < MT; t++) { acc[r][t] = 0.0f; }

        for (int s0 = 0; s0 < n_steps; s0 += U)
        {
            u32x4 w[U][R];
            uint32_t sc[U][R];
#pragma unroll
            for (int u = 0; u < U; u++)
            {
                const int k = (s0 + u) * 2048 + lane * 32;
#pragma unroll
                for (int r = 0; r < R; r++)
                {
                    w[u][r] = u32x4{ 0u, 0u, 0u, 0u };
                    sc[u][r] = 0u;
                    if constexpr (RAGGED)
                    {
                        if (k < a.K)
                        {
                            const uint8_t* wp = wrow[r] + (s0 + u) * 1024;
                            const uint8_t* sp = srow[r] + (s0 + u) * 128;
                            const u32x2 lo = __builtin_nontemporal_load((const u32x2*)wp);
                            u32x2 hi = { 0u, 0u };
                            uint32_t s_hi = 0u;
                            if (k + 32 <= a.K)
                            {
                                hi = __builtin_nontemporal_load((const u32x2*)(wp + 8));
                                s_hi = sp[1];
                            }
                            w[u][r] = u32x4{ lo[0], lo[1], hi[0], hi[1] };
                            sc[u][r] = (uint32_t)sp[0] | (s_hi << 8);
                        }
                    }
                    else if (k < a.K)
                    {
                        w[u][r] = __builtin_nontemporal_load((const u32x4*)(wrow[r] + (s0 + u) * 1024));
                        if (BLOCK == 16) { sc[u][r] = *(const uint16_t*)(srow[r] + (s0 + u) * 128); }
                        else { sc[u][r] = *(srow[r] + (s0 + u) * 64); }
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < U; u++)
            {
                if (s0 + u < n_steps)
                {
                    u32x4 x[MT][4];
#pragma unroll
                    for (int t = 0; t < MT; t++)
#pragma unroll
                        for (int p = 0; p < 4; p++) { x[t][p] = xs[(((s0 + u) * MT + t) * 4 + p) * 64 + lane]; }
#pragma unroll
                    for (int r = 0; r < R; r++)
                    {
                        const float s_lo = e4m3_byte_to_f32(sc[u][r], 0);
                        const float s_hi = BLOCK == 16 ? e4m3_byte_to_f32(sc[u][r], 1) : s_lo;
                        float part[MT][2];
#pragma unroll
                        for (int t = 0; t < MT; t++) { part[t][0] = part[t][1] = 0.0f; }
#pragma unroll
                        for (int d = 0; d < 4; d++)
                        {
                            // dword d holds elements 8d .. 8d+7; byte b holds elements 8d+2b, 8d+2b+1
                            const bf16x2 q0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[u][r][d], 1.0f, 0);
                            const bf16x2 q1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[u][r][d], 1.0f, 1);
                            const bf16x2 q2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[u][r][d], 1.0f, 2);
                            const bf16x2 q3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[u][r][d], 1.0f, 3);
#pragma unroll
                            for (int t = 0; t < MT; t++)
                            {
                                float p = part[t][d >> 1];
                                p = dot2_bf16(q0, x[t][d][0], p);
                                p = dot2_bf16(q1, x[t][d][1], p);
                                p = dot2_bf16(q2, x[t][d][2], p);
                                p = dot2_bf16(q3, x[t][d][3], p);
                                part[t][d >> 1] = p;
                            }
                        }
#pragma unroll
                        for (int t = 0; t < MT; t++)
                        {
                            acc[r][t] = fmaf(s_lo, part[t][0], acc[r][t]);
                            acc[r][t] = fmaf(s_hi, part[t][1], acc[r][t]);
                        }
                    }
                }
            }
        }

#pragma unroll
        for (int r = 0; r < R; r++)
        {
#pragma unroll
            for (int t = 0; t < MT; t++)
            {
                const float total = wave_sum(acc[r][t]);
                const int row = g * R + r;
                if (lane == 0 && row < a.n_out)
                {
                    uint16_t* y = a.Y + (long long)t * a.y_stride_tok + (long long)row * a.y_stride_out;
                    *y = finish_output(total, a.alpha, a.beta, y);
                }
            }
        }
    }
}

}    // namespace ccq

namespace ccq
{

// ------------------------------------------------------------------------------------------
// FP8 GEMV on the matrix cores, tokens 1..16 (v_mfma_f32_16x16x32_bf16).
//
// A workgroup owns RT tiles of 16 consecutive output rows and splits K over its WAVES waves in
// interleaved spans of 64 * U elements; partial 16x16 tiles meet in LDS.  Within a 64-element
// chunk lane (i = lane % 16, g = lane / 16) loads the 16 codes W[row i][chunk + 16 g ..] with one
// 128-bit load (a wave touches 16 rows x 64 contiguous bytes) and feeds two MFMAs: codes 0..7 and
// codes 8..15.  The activation operand of lane (j, g) is x[token j][chunk + 16 g ..] for the same
// two halves, so both operands agree on which k each register slot means.
//   A operand = weights: row i = output row, 8 k per lane.
//   B operand = activations: column j = token.
//   D: lane holds column j = lane % 16 (token), rows 4 g .. 4 g + 3 (output rows).
// Requires: K % 16 == 0, ldw % 16 == 0, W 16-byte aligned, ldx % 8 == 0, X 16-byte aligned.
// Static LDS: WAVES * RT * 1 KiB.

// TILED = true: a.W is the load-time repacked copy (repack_tiled_kernel), where the 16 rows x 64 codes
// of one load instruction are one contiguous KiB and consecutive k blocks follow each other.
// XLDS = true (many tokens): the activation operand takes a detour through LDS.  Fetched in operand order, the
// 16 lanes of a quarter wave read 16 different token rows -- 16 cache lines per 256 bytes, and at 16 tokens the
// kernel is bound by the L1's line rate, not by HBM (K = 12288, 4096 rows: 15.5 us against 10.4 at one token).
// Instead every wave fetches the activations of its own k span row-contiguously (eight lanes = one token's 128
// bytes of a 64-element chunk = one line), writes them to a private LDS slab and reads them back in operand
// order; both sides of the slab are conflict free (16-byte piece p of token t sits in row t % 8, slot
// 8 (t / 8) + (p ^ (t % 8)) of a 256-byte row).  No workgroup barrier: a wave only reads what it wrote.
__device__ __forceinline__ int xlds_slot(int t, int p) { return (t & 7) * 16 + ((t >> 3) * 8 + (p ^ (t & 7))); }

// AT: the 16-bit type of activations and outputs, DT_BF16 or DT_HALF (v_mfma_f32_16x16x32_f16; the weight entering a
// product is then half(decode(w) * scale), cccc/cublas_real.h:921-938).
template <int WT, int RT, int U, int WAVES, bool SCALED, bool TILED = false, bool XLDS = false, int AT = DT_BF16>
__global__ __launch_bounds__(WAVES * 64) void gemv8_mfma_kernel(const LinearArgs a)
{
    __shared__ float partial[WAVES][RT][64][4];
    __shared__ u32x4 xstage[XLDS ? WAVES * U * 128 : 1];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int i = lane & 15;
    const int g = lane >> 4;
    const int row_base = blockIdx.x * (16 * RT);
    const int last_row = a.n_out - 1;

    const uint8_t* wrow[RT];
    const int blocks_per_row = (a.K + 63) / 64;
    const int n_tiles = (a.n_out + 15) / 16;
#pragma unroll
    for (int rt = 0; rt < RT; rt++)
    {
        const int row = min(row_base + rt * 16 + i, last_row);
        if (TILED) { wrow[rt] = a.W + (long long)min(blockIdx.x * RT + rt, n_tiles - 1) * blocks_per_row * 1024 + lane * 16; }
        else { wrow[rt] = a.W + (long long)row * a.ldw + g * 16; }
    }
    const bool has_token = i < a.tokens;
    const uint16_t* xrow = a.X + (long long)(has_token ? i : 0) * a.ldx + g * 16;
    // XLDS: this lane fetches piece p (eight elements) of tokens t_fetch and t_fetch + 1 of every chunk
    const int p_fetch = lane & 7;
    const int t_fetch = ((lane >> 3) & 1) * 8 + (lane >> 4) * 2;
    u32x4* const slab = xstage + (XLDS ? wave * U * 128 : 0);

    f32x4 acc[RT];
#pragma unroll
    for (int rt = 0; rt < RT; rt++) { acc[rt] = f32x4{ 0.0f, 0.0f, 0.0f, 0.0f }; }

    const int span = 64 * U;
    // The global loads of one trip: the wave's U k-blocks of weights (one KiB per load instruction on the tiled copy) and the
    // matching activations, either in operand order (up to four tokens) or row-contiguous for the LDS detour (XLDS).
    auto issue = [&](int kb, u32x4 (&w)[U][RT], u32x4 (&x)[U][2]) {
        if constexpr (XLDS)
        {
            // activations first: loads return in issue order, and the slab can be filled while the weights are in flight
#pragma unroll
            for (int u = 0; u < U; u++)
            {
                const int k = kb + u * 64 + p_fetch * 8;
#pragma unroll
                for (int j = 0; j < 2; j++)
                {
                    x[u][j] = u32x4{ 0u, 0u, 0u, 0u };
                    if (k < a.K && t_fetch + j < a.tokens) { x[u][j] = *(const u32x4*)(a.X + (long long)(t_fetch + j) * a.ldx + k); }
                }
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++)
        {
            const int k = kb + u * 64 + g * 16;
            const bool in_k = k < a.K;
#pragma unroll
            for (int rt = 0; rt < RT; rt++)
            {
                w[u][rt] = u32x4{ 0u, 0u, 0u, 0u };
                if (in_k) { w[u][rt] = __builtin_nontemporal_load((const u32x4*)(wrow[rt] + (TILED ? (long long)(kb + u * 64) * 16 : (long long)(kb + u * 64)))); }
            }
            if constexpr (!XLDS)
            {
                x[u][0] = x[u][1] = u32x4{ 0u, 0u, 0u, 0u };
                if (in_k && has_token)
                {
                    x[u][0] = *(const u32x4*)(xrow + kb + u * 64);
                    x[u][1] = *(const u32x4*)(xrow + kb + u * 64 + 8);
                }
            }
        }
    };
    auto compute = [&](u32x4 (&w)[U][RT], u32x4 (&x)[U][2]) {
        if constexpr (XLDS)
        {
            __builtin_amdgcn_wave_barrier();         // the reads of the previous trip are done (one wave, in-order LDS)
#pragma unroll
            for (int u = 0; u < U; u++)
#pragma unroll
                for (int j = 0; j < 2; j++) { slab[u * 128 + xlds_slot(t_fetch + j, p_fetch)] = x[u][j]; }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int u = 0; u < U; u++)
#pragma unroll
                for (int h = 0; h < 2; h++) { x[u][h] = slab[u * 128 + xlds_slot(i, 2 * g + h)]; }
        }
#pragma unroll
        for (int u = 0; u < U; u++)
        {
#pragma unroll
            for (int rt = 0; rt < RT; rt++)
            {
#pragma unroll
                for (int h = 0; h < 2; h++)
                {
                    typename ActPair<AT>::type p0, p1, p2, p3;
                    fp8x4_to_pairs<WT, SCALED, AT>(w[u][rt][2 * h], a.w_scale, p0, p1);
                    fp8x4_to_pairs<WT, SCALED, AT>(w[u][rt][2 * h + 1], a.w_scale, p2, p3);
                    if constexpr (AT == DT_HALF)
                    {
                        const f16x8 wa = { p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1] };
                        acc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wa, __builtin_bit_cast(f16x8, x[u][h]), acc[rt], 0, 0, 0);
                    }
                    else
                    {
                        const bf16x8 wa = { p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1] };
                        acc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa, __builtin_bit_cast(bf16x8, x[u][h]), acc[rt], 0, 0, 0);
                    }
                }
            }
        }
    };
    // (Requesting the next trip's loads before the current trip is multiplied -- twice the bytes in flight per wave --
    // measured 5-15 % slower on every Qwen3-8B shape and token count: more waves with one trip in flight each stream better.)
    for (int kb = wave * span; kb < a.K; kb += WAVES * span)
    {
        u32x4 w[U][RT], x[U][2];
        issue(kb, w, x);
        compute(w, x);
    }

#pragma unroll
    for (int rt = 0; rt < RT; rt++)
#pragma unroll
        for (int c = 0; c < 4; c++) { partial[wave][rt][lane][c] = acc[rt][c]; }
    __syncthreads();

    for (int v = threadIdx.x; v < RT * 256; v += WAVES * 64)
    {
        const int c = v & 3;
        const int src_lane = (v >> 2) & 63;
        const int rt = v >> 8;
        float total = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES; w++) { total += partial[w][rt][src_lane][c]; }
        const int token = src_lane & 15;
        const int row = row_base + rt * 16 + 4 * (src_lane >> 4) + c;
        if (token < a.tokens && row < a.n_out)
        {
            uint16_t* y = a.Y + (long long)token * a.y_stride_tok + (long long)row * a.y_stride_out;
            *y = finish_output_act<AT>(total, a.alpha, a.beta, y);
        }
    }
}

// Builds the tiled copy of an FP8 weight [n_out][ldw]: for row tile t (16 rows) and k block b (64
// codes) the KiB at (t * ceil(K / 64) + b) * 1024 holds, at lane l = i + 16 g, the 16 codes
// W[16 t + i][64 b + 16 g ..].  Rows beyond n_out and codes beyond K are zero.
static __global__ __launch_bounds__(256) void repack_tiled_kernel(const uint8_t* __restrict__ W, uint8_t* __restrict__ dst, int n_out, int K, long long ldw)
{
    const int blocks_per_row = (K + 63) / 64;
    const long long n_chunks = (long long)((n_out + 15) / 16) * blocks_per_row * 64;
    for (long long c = (long long)blockIdx.x * 256 + threadIdx.x; c < n_chunks; c += (long long)gridDim.x * 256)
    {
        const int l = (int)(c & 63);
        const long long blk = c >> 6;
        const int b = (int)(blk % blocks_per_row);
        const int row = (int)(blk / blocks_per_row) * 16 + (l & 15);
        const int k = b * 64 + (l >> 4) * 16;
        u32x4 v = { 0u, 0u, 0u, 0u };
        if (row < n_out && k < K) { v = *(const u32x4*)(W + (long long)row * ldw + k); }
        *(u32x4*)(dst + c * 16) = v;
    }
}

// ------------------------------------------------------------------------------------------
// FP4 block-scale GEMV on the matrix cores over a load-time tiled copy, tokens 1..16.
//
// fp4 * e4m3 is exact in BF16, but the hardware conversion only applies a power-of-two scale, so the block scale is
// kept out of the operand: one v_mfma_f32_16x16x16_bf16 contracts exactly one 16-element scale block of 16 rows
// against up to 16 tokens (FP32 sums of exact products), and the result is multiplied by the rows' block scales
// and added to the accumulators.  For that the weight is the COLUMN operand: the output lane (n = lane % 16, g)
// holds row n for tokens 4 g .. 4 g + 3 and needs one scale per instruction -- its own row's.
//   A operand (rows)    = tokens:      lane (j, g) holds x[j][block + 4 g .. + 3]
//   B operand (columns) = weight rows: lane (n, g) holds w[n][block + 4 g .. + 3]
// Tiled copy (repack_tiled_fp4_kernel), per row tile t (16 rows) and chunk c (128 elements):
//   codes   KiB (t * chunks + c): lane l = n + 16 g owns 16 bytes; byte pair m = 0..7 holds the four nibbles of
//           row 16 t + n, elements 128 c + 16 m + 4 g .. + 3 (low nibble first, as in the file)
//   scales  after all code KiBs, 16 * (128 / BLOCK) bytes per (t, c): row n's scales of the chunk, in order
// so a wave reads one contiguous KiB of codes and one contiguous 128 (64) bytes of scales per chunk.
// A workgroup owns RT row tiles and splits K over its waves in spans of 128 * U elements; every wave fetches the
// activations of its span row-contiguously and turns them into operand order through a private LDS slab (8-byte
// piece q of token t sits at piece q ^ 2 t of the token's 256-byte row: conflict free both ways).
// MT = 4 or 16: tokens the slab and the fetch are sized for.  K % 32 == 0, X 16-byte aligned, ldx % 8 == 0.
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) short s16x4;        // operand type of the 16x16x16 BF16 matrix-core builtin

template <int BLOCK, int RT, int U, int WAVES, int MT>
__global__ __launch_bounds__(WAVES * 64) void gemv4_mfma_kernel(const LinearArgs a, const uint8_t* __restrict__ tiled_scales)
{
    static_assert(BLOCK == 16 || BLOCK == 32, "block scale length");
    static_assert(MT == 4 || MT == 16, "token group");
    constexpr int NS = 128 / BLOCK;                        // scale bytes per row and chunk
    __shared__ float partial[WAVES][RT][64][4];
    __shared__ u32x2 xstage[WAVES * U * MT * 32];          // per wave and chunk: MT token rows of 32 8-byte pieces

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n = lane & 15;
    const int g = lane >> 4;
    const int chunks = (a.K + 127) / 128;
    const int n_tiles = (a.n_out + 15) / 16;
    const int row_base = blockIdx.x * (16 * RT);

    const uint8_t* wtile[RT];
    const uint8_t* stile[RT];
#pragma unroll
    for (int rt = 0; rt < RT; rt++)
    {
        const long long tile = min((int)blockIdx.x * RT + rt, n_tiles - 1);      // a clamped tile is computed and dropped
        wtile[rt] = a.W + tile * chunks * 1024 + lane * 16;
        stile[rt] = tiled_scales + tile * chunks * (16 * NS) + n * NS;
    }
    u32x2* const slab = xstage + wave * (U * MT * 32);
    const int xk = (lane & 15) * 8;                         // element offset of this lane's 16 bytes within a chunk row
    const int xt = lane >> 4;                               // token of the first fetch; + 4 per further fetch

    f32x4 acc[RT];
#pragma unroll
    for (int rt = 0; rt < RT; rt++) { acc[rt] = f32x4{ 0.0f, 0.0f, 0.0f, 0.0f }; }
    const f32x4 zero = { 0.0f, 0.0f, 0.0f, 0.0f };

    const int span = 128 * U;
    for (int kb = wave * span; kb < a.K; kb += WAVES * span)
    {
        u32x4 xr[U][MT / 4];
        u32x4 w[U][RT];
        u32x2 sc[U][RT];
#pragma unroll
        for (int u = 0; u < U; u++)
        {
            const int k = kb + u * 128 + xk;
#pragma unroll
            for (int j = 0; j < MT / 4; j++)
            {
                xr[u][j] = u32x4{ 0u, 0u, 0u, 0u };
                if (k < a.K && xt + 4 * j < a.tokens) { xr[u][j] = *(const u32x4*)(a.X + (long long)(xt + 4 * j) * a.ldx + k); }
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++)
        {
            const long long chunk = kb / 128 + u;
            const bool in_k = kb + u * 128 < a.K;
#pragma unroll
            for (int rt = 0; rt < RT; rt++)
            {
                w[u][rt] = u32x4{ 0u, 0u, 0u, 0u };
                sc[u][rt] = u32x2{ 0u, 0u };
                if (in_k)
                {
                    w[u][rt] = __builtin_nontemporal_load((const u32x4*)(wtile[rt] + chunk * 1024));
                    if (NS == 8) { sc[u][rt] = *(const u32x2*)(stile[rt] + chunk * (16 * NS)); }
                    else { sc[u][rt][0] = *(const uint32_t*)(stile[rt] + chunk * (16 * NS)); }
                }
            }
        }
        __builtin_amdgcn_wave_barrier();                   // the reads of the previous trip are done (one wave, in-order LDS)
#pragma unroll
        for (int u = 0; u < U; u++)
#pragma unroll
            for (int j = 0; j < MT / 4; j++)
            {
                const int t = xt + 4 * j;
                *(u32x4*)&slab[(u * MT + t) * 32 + ((2 * (lane & 15)) ^ ((2 * t) & 31))] = xr[u][j];
            }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int u = 0; u < U; u++)
        {
#pragma unroll
            for (int m = 0; m < 8; m++)
            {
                u32x2 xv = { 0u, 0u };
                if (MT == 16 || n < MT) { xv = slab[(u * MT + (MT == 16 ? n : (n & (MT - 1)))) * 32 + ((4 * m + g) ^ ((2 * n) & 31))]; }
                const s16x4 xa = __builtin_bit_cast(s16x4, xv);
#pragma unroll
                for (int rt = 0; rt < RT; rt++)
                {
                    const uint32_t word = w[u][rt][m >> 1];
                    const bf16x2 lo = (m & 1) ? __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(word, 1.0f, 2) : __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(word, 1.0f, 0);
                    const bf16x2 hi = (m & 1) ? __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(word, 1.0f, 3) : __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(word, 1.0f, 1);
                    const bf16x4 wv = { lo[0], lo[1], hi[0], hi[1] };
                    const f32x4 t = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(xa, __builtin_bit_cast(s16x4, wv), zero, 0, 0, 0);
                    const int si = BLOCK == 16 ? m : (m >> 1);                  // scale byte of this block within the chunk
                    const uint32_t sword = sc[u][rt][si >> 2];
                    float s;
                    switch (si & 3)
                    {
                    case 0: s = __builtin_amdgcn_cvt_f32_fp8(sword, 0); break;
                    case 1: s = __builtin_amdgcn_cvt_f32_fp8(sword, 1); break;
                    case 2: s = __builtin_amdgcn_cvt_f32_fp8(sword, 2); break;
                    default: s = __builtin_amdgcn_cvt_f32_fp8(sword, 3); break;
                    }
#pragma unroll
                    for (int c = 0; c < 4; c++) { acc[rt][c] = fmaf(s, t[c], acc[rt][c]); }
                }
            }
        }
    }

#pragma unroll
    for (int rt = 0; rt < RT; rt++)
#pragma unroll
        for (int c = 0; c < 4; c++) { partial[wave][rt][lane][c] = acc[rt][c]; }
    __syncthreads();

    // D: lane (n, g) holds weight row n for tokens 4 g .. 4 g + 3
    for (int v = threadIdx.x; v < RT * 256; v += WAVES * 64)
    {
        const int src_lane = v & 63;
        const int c = (v >> 6) & 3;
        const int rt = v >> 8;
        float total = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES; w++) { total += partial[w][rt][src_lane][c]; }
        const int token = 4 * (src_lane >> 4) + c;
        const int row = row_base + rt * 16 + (src_lane & 15);
        if (token < a.tokens && row < a.n_out)
        {
            uint16_t* y = a.Y + (long long)token * a.y_stride_tok + (long long)row * a.y_stride_out;
            *y = finish_output(total, a.alpha, a.beta, y);
        }
    }
}

// Builds the tiled copy of an FP4 weight (layout above) from the packed codes W [n_out][K / 2] and the block scales
// S over the flat element index.  One thread per 16 destination bytes of codes; the scales of a (tile, chunk) are
// written by its first 16 * NS threads... here: by the thread that owns lane n, g == 0.
static __global__ __launch_bounds__(256) void repack_tiled_fp4_kernel(const uint8_t* __restrict__ W, const uint8_t* __restrict__ S, uint8_t* __restrict__ dst,
                                                              int n_out, int K, int block)
{
    const int chunks = (K + 127) / 128;
    const int ns = 128 / block;
    const long long n_units = (long long)((n_out + 15) / 16) * chunks * 64;
    uint8_t* const dst_scales = dst + (long long)((n_out + 15) / 16) * chunks * 1024;
    for (long long q = (long long)blockIdx.x * 256 + threadIdx.x; q < n_units; q += (long long)gridDim.x * 256)
    {
        const int l = (int)(q & 63);
        const long long tc = q >> 6;                        // tile * chunks + chunk
        const int c = (int)(tc % chunks);
        const int row = (int)(tc / chunks) * 16 + (l & 15);
        const int g = l >> 4;
        uint16_t out[8];
#pragma unroll
        for (int m = 0; m < 8; m++)
        {
            const int k = 128 * c + 16 * m + 4 * g;
            out[m] = (row < n_out && k < K) ? *(const uint16_t*)(W + (((long long)row * K + k) >> 1)) : (uint16_t)0;
        }
        u32x4 v;
#pragma unroll
        for (int d = 0; d < 4; d++) { v[d] = (uint32_t)out[2 * d] | ((uint32_t)out[2 * d + 1] << 16); }
        *(u32x4*)(dst + q * 16) = v;
        if (g == 0)
        {
            for (int i = 0; i < ns; i++)
            {
                const int k = 128 * c + block * i;
                dst_scales[tc * (16 * ns) + (l & 15) * ns + i] = (row < n_out && k < K) ? S[((long long)row * K + k) / block] : (uint8_t)0;
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// Fallback for any layout / type / size the fast kernels do not take: one lane per output element,
// software decode of the flat element index exactly as the reference's dequant kernels index it.
//   element (o, k) of the weight is at flat index  o * w_stride_out + k * w_stride_k
//   element (t, k) of the activation is at         t * x_stride_tok + k * x_stride_k
struct GenericArgs
{
    const uint8_t* W;
    const uint8_t* blk_sc;
    const uint16_t* X;
    uint16_t* Y;
    long long w_stride_out, w_stride_k, x_stride_tok, x_stride_k, y_stride_tok, y_stride_out;
    int n_out, tokens, K, w_type;
    int act_type;              // DT_BF16 or DT_HALF: type of X and Y, and the rounding of the dequantised weight
    unsigned block_size;
    float w_scale, alpha, beta;
};

static __global__ __launch_bounds__(256) void generic_linear_kernel(const GenericArgs a)
{
    const long long total = (long long)a.n_out * a.tokens;
    for (long long idx = (long long)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (long long)gridDim.x * 256)
    {
        const int o = (int)(idx % a.n_out);
        const int t = (int)(idx / a.n_out);
        float acc = 0.0f;
        for (int k = 0; k < a.K; k++)
        {
            const long long fi = (long long)o * a.w_stride_out + (long long)k * a.w_stride_k;
            float wv;
            if (a.w_type == DT_FP4)
            {
                const uint32_t byte = a.W[fi >> 1];
                const float s = a.blk_sc ? e4m3_to_f32(a.blk_sc[fi / a.block_size]) : a.w_scale;
                wv = fp4_to_f32((fi & 1) ? (byte >> 4) : (byte & 0xFu)) * s;
            }
            else
            {
                wv = (a.w_type == DT_E5M2 ? e5m2_to_f32(a.W[fi]) : e4m3_to_f32(a.W[fi])) * a.w_scale;
            }
            const uint32_t xb = a.X[(long long)t * a.x_stride_tok + (long long)k * a.x_stride_k];
            const bool half = a.act_type == DT_HALF;
            const float wq = half ? half_bits_to_f32(f32_to_half_bits(wv)) : bf16_bits_to_f32(f32_to_bf16_bits(wv));
            acc = fmaf(wq, half ? half_bits_to_f32(xb) : bf16_bits_to_f32(xb), acc);
        }
        uint16_t* y = a.Y + (long long)t * a.y_stride_tok + (long long)o * a.y_stride_out;
        *y = a.act_type == DT_HALF ? finish_output_act<DT_HALF>(acc, a.alpha, a.beta, y) : finish_output(acc, a.alpha, a.beta, y);
    }
}

}    // namespace ccq
