// Variants of the register-fed FP8 prefill GEMM (csrc/gemm_kernels.h: gemm_mfma_direct_kernel on the tiled copy) that were
// measured against it and not adopted, kept runnable so that the measurements can be repeated (bench.py --workload
// prefill_variants).  Built into libcccc_bench.so, which only bench.py loads; the product library does not carry them.
//   MEMSPREAD  one memory instruction per token block (the order the product kernel adopted from here); without it the
//           weight loads follow the barrier in one burst and the stores and activation loads sit together mid-tile
//   SPREAD  the FP8 -> BF16 conversions issued between the matrix-core instructions (the high halves of tile kt while
//           its first step is multiplied, the low halves of tile kt + 1 during its second step) instead of in a block
//           in front of the k-tile's barrier
//   RAST    every XCD (workgroup index % 8) owns a block of (token tiles / P) x (feature tiles / Q), P * Q = 8, instead
//           of "feature tile n on XCD n % 8 with every token tile"
//   TRACE   wave 0 of every workgroup adds up the clock ticks it spends (a) converting, which includes the wait for the
//           weight bytes, (b) at the k-tile's barrier and (c) between the barrier and the end of the k-tile
// Everything else -- tile shapes, operand layouts, LDS swizzle, prefetch distances, epilogue -- is the product kernel's.
// gemm_ablation_kernel: the k-tile's ingredients one by one on operands that need no HBM.
#include "../csrc/gemm_kernels.h"
#include "../../include/cccc_hip_quant.h"
#include <hip/hip_runtime.h>

namespace
{

using namespace ccq;

__device__ __forceinline__ unsigned long long ticks()
{
    __builtin_amdgcn_sched_barrier(0);
    const unsigned long long t = __builtin_readcyclecounter();
    __builtin_amdgcn_sched_barrier(0);
    return t;
}

struct Raster
{
    int P, Q;
};

template <bool SCALED, int MB, bool SPLIT, int NB, bool SPREAD, bool RAST, bool TRACE, int MEMSPREAD = 0>
__global__ __launch_bounds__(256, 2) void gemm_variant_kernel(const LinearArgs a, const int n_tiles, const int m_tiles, float* __restrict__ partial,
                                                              const Raster rast, unsigned long long* __restrict__ trace)
{
    constexpr int WT = DT_E5M2;
    constexpr int BTOK = MB * 16;
    constexpr int BK = 64, CPR = 8;
    constexpr int X_PER_THREAD = BTOK * CPR / 256;
    __shared__ u32x4 xs[2][BTOK * CPR];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int n_tile, m_tile;
    if constexpr (!RAST)
    {
        const int n_pad = (n_tiles + 7) & ~7;
        n_tile = blockIdx.x % n_pad;
        m_tile = blockIdx.x / n_pad;
        if (n_tile >= n_tiles) { return; }
    }
    else
    {
        const int x = blockIdx.x & 7, j = blockIdx.x >> 3;
        const int bm = (m_tiles + rast.P - 1) / rast.P, bn = (n_tiles + rast.Q - 1) / rast.Q;
        m_tile = (x / rast.Q) * bm + j % bm;
        n_tile = (x % rast.Q) * bn + j / bm;
        if (j / bm >= bn || m_tile >= m_tiles || n_tile >= n_tiles) { return; }
    }
    const int out_base = n_tile * (64 * NB) + wave * (16 * NB);
    const int tok_base = m_tile * BTOK;
    const int i16 = lane & 15;
    const int g = lane >> 4;
    const int n_kt_total = a.K / BK;
    const int kt_begin = SPLIT ? (int)((long long)n_kt_total * blockIdx.y / gridDim.y) : 0;
    const int n_kt = SPLIT ? (int)((long long)n_kt_total * (blockIdx.y + 1) / gridDim.y) - kt_begin : n_kt_total;
    const uint8_t* const w_begin = a.W + (long long)kt_begin * 1024;
    const uint8_t* const x_begin = (const uint8_t*)a.X + (long long)kt_begin * BK * 2;

    f32x4 acc[MB][NB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++) { acc[mb][nb] = f32x4{ 0.0f, 0.0f, 0.0f, 0.0f }; }

    long long w_tile_base[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) { w_tile_base[nb] = (long long)min(out_base / 16 + nb, (a.n_out + 15) / 16 - 1) * n_kt_total * 1024; }
    const uint32_t w_off = lane * 16;
    uint32_t x_off[X_PER_THREAD];
    int x_store[X_PER_THREAD];
#pragma unroll
    for (int i = 0; i < X_PER_THREAD; i++)
    {
        const int q = tid + i * 256;
        x_off[i] = (uint32_t)(((long long)min(tok_base + q / CPR, a.tokens - 1) * a.ldx + (q % CPR) * 8) * 2);
        x_store[i] = (q / CPR) * CPR + swizzled_chunk_n<CPR>(q / CPR, q % CPR);
    }

    u32x4 wraw[2][NB], xreg[X_PER_THREAD];
    auto fetch_x = [&](int kt) {
        const int k0 = min(kt, n_kt - 1) * BK;
#pragma unroll
        for (int i = 0; i < X_PER_THREAD; i++) { xreg[i] = *(const u32x4*)(x_begin + (size_t)k0 * 2 + (size_t)x_off[i]); }
    };
    auto fetch_w = [&](int kt, u32x4* wr) {
        const int k0 = min(kt, n_kt - 1) * 1024;
#pragma unroll
        for (int nb = 0; nb < NB; nb++) { wr[nb] = *(const u32x4*)(w_begin + w_tile_base[nb] + k0 + (size_t)w_off); }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int i = 0; i < X_PER_THREAD; i++) { xs[buf][x_store[i]] = xreg[i]; }
    };
    // half h (0: bytes 0..7, 1: bytes 8..15) of a raw 16-byte weight piece -> the lane's operand of matrix-core step h
    auto cvt_half = [&](const u32x4& raw, int h, u32x4& out) {
#pragma unroll
        for (int d = 0; d < 2; d++)
        {
            bf16x2 p, q;
            fp8x4_to_bf16<WT, SCALED>(raw[2 * h + d], a.w_scale, p, q);
            out[2 * d] = __builtin_bit_cast(uint32_t, p);
            out[2 * d + 1] = __builtin_bit_cast(uint32_t, q);
        }
    };

    unsigned long long t_cvt = 0, t_bar = 0, t_mma = 0, t_begin = 0;
    if constexpr (TRACE) { t_begin = ticks(); }

    u32x4 wf[2][NB];
    constexpr int AHEAD = 3, FRAGS = 2 * MB;
    constexpr int CVT_OPS = SCALED ? 16 : 4;         // VALU instructions of one half-piece conversion
    auto k_tile = [&](int kt, u32x4* wcur, u32x4* wnext) {
        unsigned long long c0 = 0, c1 = 0, c2 = 0;
        if constexpr (TRACE) { c0 = ticks(); }
        if constexpr (!SPREAD)
        {
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
            {
                cvt_half(wcur[nb], 0, wf[0][nb]);
                cvt_half(wcur[nb], 1, wf[1][nb]);
            }
        }
        if constexpr (TRACE)
        {
            asm volatile("" ::"v"(wf[0][0][0]), "v"(wf[1][NB - 1][3]));       // the conversions (and the wait for their bytes) end here
            c1 = ticks();
        }
        __syncthreads();
        if constexpr (TRACE) { c2 = ticks(); }
        if constexpr (!SPREAD && MEMSPREAD == 0) { fetch_w(kt + 1, wnext); }
        const u32x4* xt = xs[kt & 1];
        auto read_frag = [&](int f) {
            const int row = (f % MB) * 16 + i16;
            return xt[row * CPR + swizzled_chunk_n<CPR>(row, 2 * g + f / MB)];
        };
        u32x4 ring[AHEAD + 1];
#pragma unroll
        for (int f = 0; f < AHEAD; f++) { ring[f] = read_frag(f); }
#pragma unroll
        for (int f = 0; f < FRAGS; f++)
        {
            if constexpr (SPREAD) { __builtin_amdgcn_sched_barrier(0); }
            if constexpr (MEMSPREAD != 0)
            {
                // one memory instruction per token block.  1: the weight pieces with the first blocks, the stores from the
                // middle on, each activation load one block behind the store that frees its register; 2: weights, stores
                // and loads each spread over the whole k-tile; 3: weights first, stores and loads spread over the whole k-tile
                constexpr int WS = MEMSPREAD == 2 ? FRAGS / NB : 1;
                constexpr int S0 = MEMSPREAD == 1 ? FRAGS / 2 : 2, SS = MEMSPREAD == 1 ? 1 : 4;
                if (f % WS == 0 && f / WS < NB)
                {
                    const int k0 = min(kt + 1, n_kt - 1) * 1024;
                    wnext[f / WS] = *(const u32x4*)(w_begin + w_tile_base[f / WS] + k0 + (size_t)w_off);
                }
                if (f >= S0 && (f - S0) % SS == 0 && (f - S0) / SS < X_PER_THREAD) { xs[(kt + 1) & 1][x_store[(f - S0) / SS]] = xreg[(f - S0) / SS]; }
                if (f >= S0 + 1 && (f - S0 - 1) % SS == 0 && (f - S0 - 1) / SS < X_PER_THREAD)
                {
                    const int i = (f - S0 - 1) / SS;
                    xreg[i] = *(const u32x4*)(x_begin + (size_t)(min(kt + 2, n_kt - 1) * BK) * 2 + (size_t)x_off[i]);
                }
            }
            if (MEMSPREAD == 0 && f == FRAGS / 2)
            {
                stage((kt + 1) & 1);
                fetch_x(kt + 2);
                if constexpr (SPREAD)
                {
                    fetch_w(kt + 2, wcur);       // the raw bytes of tile kt are all converted by now
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            if (f + AHEAD < FRAGS) { ring[(f + AHEAD) % (AHEAD + 1)] = read_frag(f + AHEAD); }
            const bf16x8 xf = __builtin_bit_cast(bf16x8, ring[f % (AHEAD + 1)]);
            const int s = f / MB, mb = f % MB;
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
            {
                acc[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wf[s][nb]), xf, acc[mb][nb], 0, 0, 0);
            }
            if constexpr (SPREAD)
            {
                // this token block's share of the conversions
                const int p_begin = mb * NB / MB, p_end = (mb + 1) * NB / MB;
#pragma unroll
                for (int p = p_begin; p < p_end; p++)
                {
                    if (s == 0) { cvt_half(wcur[p], 1, wf[1][p]); }
                    else { cvt_half(wnext[p], 0, wf[0][p]); }
                }
                if (f + AHEAD < FRAGS) { __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); }
                constexpr int PER = (((NB + MB - 1) / MB) * CVT_OPS + NB - 1) / NB;
#pragma unroll
                for (int nb = 0; nb < NB; nb++)
                {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, PER, 0);
                }
            }
        }
        if constexpr (SPREAD) { __builtin_amdgcn_sched_barrier(0); }
        else if constexpr (MEMSPREAD != 0)
        {
            constexpr int WS = MEMSPREAD == 2 ? FRAGS / NB : 1;
            constexpr int S0 = MEMSPREAD == 1 ? FRAGS / 2 : 2, SS = MEMSPREAD == 1 ? 1 : 4;
            static_assert(S0 + 1 + (X_PER_THREAD - 1) * SS < FRAGS && (NB - 1) * WS < FRAGS, "spread slots");
            __builtin_amdgcn_sched_group_barrier(0x100, AHEAD, 0);
#pragma unroll
            for (int f = 0; f < FRAGS; f++)
            {
                if (f % WS == 0 && f / WS < NB) { __builtin_amdgcn_sched_group_barrier(0x020, 1, 0); }
                if (f >= S0 && (f - S0) % SS == 0 && (f - S0) / SS < X_PER_THREAD) { __builtin_amdgcn_sched_group_barrier(0x200, 1, 0); }
                if (f >= S0 + 1 && (f - S0 - 1) % SS == 0 && (f - S0 - 1) / SS < X_PER_THREAD) { __builtin_amdgcn_sched_group_barrier(0x020, 1, 0); }
                if (f + AHEAD < FRAGS) { __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); }
                __builtin_amdgcn_sched_group_barrier(0x008, NB, 0);
            }
        }
        else
        {
            __builtin_amdgcn_sched_group_barrier(0x020, NB, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, AHEAD, 0);
#pragma unroll
            for (int f = 0; f < FRAGS; f++)
            {
                if (f == FRAGS / 2)
                {
                    __builtin_amdgcn_sched_group_barrier(0x200, X_PER_THREAD, 0);
                    __builtin_amdgcn_sched_group_barrier(0x020, X_PER_THREAD, 0);
                }
                if (f + AHEAD < FRAGS) { __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); }
                __builtin_amdgcn_sched_group_barrier(0x008, NB, 0);
            }
        }
        if constexpr (TRACE)
        {
            const unsigned long long c3 = ticks();
            t_cvt += c1 - c0;
            t_bar += c2 - c1;
            t_mma += c3 - c2;
        }
    };

    fetch_x(0);
    fetch_w(0, wraw[0]);
    if constexpr (SPREAD) { fetch_w(1, wraw[1]); }
    stage(0);
    fetch_x(1);
    if constexpr (SPREAD)
    {
#pragma unroll
        for (int nb = 0; nb < NB; nb++) { cvt_half(wraw[0][nb], 0, wf[0][nb]); }
    }
    for (int kt = 0; kt < n_kt; kt += 2)
    {
        k_tile(kt, wraw[0], wraw[1]);
        if (kt + 1 < n_kt) { k_tile(kt + 1, wraw[1], wraw[0]); }
    }
    if constexpr (TRACE)
    {
        if (tid == 0)
        {
            const unsigned long long t_end = ticks();
            const size_t wg = (size_t)blockIdx.y * gridDim.x + blockIdx.x;
            trace[wg * 4 + 0] = t_cvt;
            trace[wg * 4 + 1] = t_bar;
            trace[wg * 4 + 2] = t_mma;
            trace[wg * 4 + 3] = t_end - t_begin;
        }
    }

#pragma unroll
    for (int mb = 0; mb < MB; mb++)
    {
        const int tok = tok_base + mb * 16 + i16;
        if (tok >= a.tokens) { continue; }
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
        {
            const int out = out_base + nb * 16 + 4 * g;
            if (out + 3 >= a.n_out) { continue; }           // (the benchmark shapes are multiples of the tile)
            const f32x4 r = acc[mb][nb];
            if constexpr (SPLIT) { *(f32x4*)(partial + ((long long)blockIdx.y * a.tokens + tok) * a.n_out + out) = r; }
            else
            {
                uint16_t o[4];
#pragma unroll
                for (int v = 0; v < 4; v++) { o[v] = finish_output_act<DT_BF16>(r[v], a.alpha, 0.0f, nullptr); }
                *(uint2*)(a.Y + (long long)tok * a.y_stride_tok + out) = uint2{ (uint32_t)o[0] | ((uint32_t)o[1] << 16), (uint32_t)o[2] | ((uint32_t)o[3] << 16) };
            }
        }
    }
}

template <bool SCALED, int MB, bool SPLIT, int NB, bool SPREAD, bool RAST, bool TRACE, int MEMSPREAD = 0>
void launch_variant(const LinearArgs& a, int splits, float* partial, unsigned long long* trace, unsigned* n_wgs)
{
    const int n_tiles = (a.n_out + 64 * NB - 1) / (64 * NB);
    const int m_tiles = (a.tokens + MB * 16 - 1) / (MB * 16);
    const Raster rast = { 4, 2 };
    const unsigned gx = RAST ? 8u * ((m_tiles + rast.P - 1) / rast.P) * ((n_tiles + rast.Q - 1) / rast.Q) : (unsigned)(((n_tiles + 7) & ~7) * m_tiles);
    *n_wgs = gx * (unsigned)splits;
    gemm_variant_kernel<SCALED, MB, SPLIT, NB, SPREAD, RAST, TRACE, MEMSPREAD><<<dim3(gx, splits), 256, 0, nullptr>>>(a, n_tiles, m_tiles, partial, rast, trace);
    if (SPLIT) { launch_splitk_combine<DT_BF16>(partial, splits, a, nullptr); }
}

// tile: 0 = 128 tokens x 256 features, 1 = 64 x 192, 2 = 128 x 256 with the k range split in four, 3 = 64 x 256,
// 4 = 128 x 192, 5 = 128 x 256 split in two, 6 = 64 x 256 split in two
// the memory instructions of a k-tile one per token block (tiles 0, 1, 3, 4 and the k split of 4)
template <int MODE>
bool launch_tile_memspread(int tile, const LinearArgs& a, float* partial, unsigned* n_wgs)
{
    switch (tile)
    {
    case 0: launch_variant<false, 8, false, 4, false, false, false, MODE>(a, 1, partial, nullptr, n_wgs); return true;
    case 1: launch_variant<false, 4, false, 3, false, false, false, MODE>(a, 1, partial, nullptr, n_wgs); return true;
    case 2: launch_variant<false, 8, true, 4, false, false, false, MODE>(a, 4, partial, nullptr, n_wgs); return true;
    case 3: launch_variant<false, 4, false, 4, false, false, false, MODE>(a, 1, partial, nullptr, n_wgs); return true;
    case 4: launch_variant<false, 8, false, 3, false, false, false, MODE>(a, 1, partial, nullptr, n_wgs); return true;
    default: return false;
    }
}

template <bool SPREAD, bool RAST, bool TRACE>
bool launch_tile(int tile, bool scaled, const LinearArgs& a, float* partial, unsigned long long* trace, unsigned* n_wgs)
{
    if (scaled)
    {
        if (tile != 0 || RAST || TRACE) { return false; }
        launch_variant<true, 8, false, 4, SPREAD, false, false>(a, 1, partial, trace, n_wgs);
        return true;
    }
    switch (tile)
    {
    case 0: launch_variant<false, 8, false, 4, SPREAD, RAST, TRACE>(a, 1, partial, trace, n_wgs); return true;
    case 1: launch_variant<false, 4, false, 3, SPREAD, RAST, TRACE>(a, 1, partial, trace, n_wgs); return true;
    case 2: launch_variant<false, 8, true, 4, SPREAD, RAST, TRACE>(a, 4, partial, trace, n_wgs); return true;
    case 3: launch_variant<false, 4, false, 4, SPREAD, RAST, TRACE>(a, 1, partial, trace, n_wgs); return true;
    case 4: launch_variant<false, 8, false, 3, SPREAD, RAST, TRACE>(a, 1, partial, trace, n_wgs); return true;
    case 5: launch_variant<false, 8, true, 4, SPREAD, RAST, TRACE>(a, 2, partial, trace, n_wgs); return true;
    case 6: launch_variant<false, 4, true, 4, SPREAD, RAST, TRACE>(a, 2, partial, trace, n_wgs); return true;
    default: return false;
    }
}

// What the k-tile of the 128 x 256 tile costs piece by piece: its 64 matrix-core instructions per wave (32 accumulator
// blocks, two workgroups per CU) on operands that never leave the registers, then with the other ingredients of the
// product loop switched on one by one (FLAGS):
//   1  CVT   the k-tile's sixteen FP8 -> BF16 dword conversions, on raw words that change every trip
//   2  LDSR  the sixteen activation fragments read from LDS, three instructions ahead of their use, as the product does
//   4  BAR   the workgroup barrier of the k-tile
//   8  LDSW  the four 16-byte stores per thread of the next activation tile
//   16 GW    the four 16-byte weight loads per lane (KiB-contiguous per wave, from a 4 MiB window that stays in L2)
//   32 GX    the four 16-byte activation loads per thread (from a 1 MiB window)
// No result is meaningful; the operands are finite and the accumulators are kept alive by a store that never happens.
// SCHED: 0 = memory instructions in bursts (the weight loads behind the barrier, the stores and the activation loads in
// the middle of the k-tile); bit 0 = the four stores one per token block from the middle on; bit 1 = the four weight
// loads one per token block from the start on; bit 2 = the activation loads one per token block behind the stores;
// 7 = the product kernel's order.  AHEAD: fragments read ahead of their use.
template <int FLAGS, int AHEAD, int SCHED, int WS = 1, int S0 = 8, int SS = 1>
__device__ __forceinline__ void gemm_ablation_body(const int trips, const uint32_t seed, const uint8_t* __restrict__ wbuf,
                                                   const uint8_t* __restrict__ xbuf, float* __restrict__ sink)
{
    constexpr bool CVT = FLAGS & 1, LDSR = FLAGS & 2, BAR = FLAGS & 4, LDSW = FLAGS & 8, GW = FLAGS & 16, GX = FLAGS & 32;
    constexpr int MB = 8, NB = 4, CPR = 8, BTOK = 128, X_PER_THREAD = 4, FRAGS = 2 * MB;
    constexpr bool ST1 = SCHED & 1, WL1 = SCHED & 2, XL1 = SCHED & 4;
    __shared__ u32x4 xs[2][BTOK * CPR];
    const int tid = threadIdx.x, lane = tid & 63, i16 = lane & 15, g = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    f32x4 acc[MB][NB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++) { acc[mb][nb] = f32x4{ 0.0f, 0.0f, 0.0f, 0.0f }; }
    u32x4 raw[NB], wf[2][NB], xreg[X_PER_THREAD], xconst[4];
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
    {
        const uint32_t r = (seed + tid * 7u + nb) & 0x3b3b3b3bu;           // small finite E5M2 codes
        raw[nb] = u32x4{ r, r ^ 0x01010101u, r ^ 0x02020202u, r ^ 0x03030303u };
        wf[0][nb] = u32x4{ 0x3c003c00u, 0x3c003c00u, 0x3c003c00u, 0x3c003c00u };
        wf[1][nb] = wf[0][nb];
    }
#pragma unroll
    for (int i = 0; i < 4; i++)
    {
        xconst[i] = u32x4{ 0x3a003a00u + i, 0x3a003a00u, 0x3a003a00u, 0x3a003a00u };
        xreg[i] = xconst[i];
    }
    int x_store[X_PER_THREAD];
#pragma unroll
    for (int i = 0; i < X_PER_THREAD; i++)
    {
        const int q = tid + i * 256;
        x_store[i] = (q / CPR) * CPR + swizzled_chunk_n<CPR>(q / CPR, q % CPR);
        xs[0][x_store[i]] = xconst[i];
        xs[1][x_store[i]] = xconst[i];
    }
    __syncthreads();
    const uint8_t* const w_wave = wbuf + (size_t)((blockIdx.x * 4 + wave) & 15) * (256 << 10) + (size_t)lane * 16;      // 16 windows of 256 KiB
    const uint8_t* const x_wg = xbuf + (size_t)(blockIdx.x & 7) * (128 << 10) + (size_t)tid * 16;                     // 8 windows of 128 KiB
    for (int t = 0; t < trips; t++)
    {
        if constexpr (CVT)
        {
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
            {
                if constexpr (!GW) { raw[nb][0] ^= (uint32_t)(t & 1); }
#pragma unroll
                for (int d = 0; d < 4; d++)
                {
                    bf16x2 p, q;
                    fp8x4_to_bf16<DT_E5M2, false>(raw[nb][d] & 0x3b3b3b3bu, 1.0f, p, q);
                    wf[d / 2][nb][2 * (d & 1)] = __builtin_bit_cast(uint32_t, p);
                    wf[d / 2][nb][2 * (d & 1) + 1] = __builtin_bit_cast(uint32_t, q);
                }
            }
        }
        if constexpr (BAR) { __syncthreads(); }
        u32x4 rawn[NB];
        auto load_w = [&](int nb) { rawn[nb] = *(const u32x4*)(w_wave + (size_t)(((t + 1) & 15) * NB + nb) * 4096 + (size_t)(nb * 1024)); };
        auto store_x = [&](int i) { xs[(t + 1) & 1][x_store[i]] = xreg[i] & u32x4{ 0x3b7f3b7fu, 0x3b7f3b7fu, 0x3b7f3b7fu, 0x3b7f3b7fu }; };
        auto load_x = [&](int i) { xreg[i] = *(const u32x4*)(x_wg + (size_t)((t + 2) & 7) * 16384 + (size_t)i * 4096); };
        if constexpr (GW && !WL1)
        {
#pragma unroll
            for (int nb = 0; nb < NB; nb++) { load_w(nb); }
        }
        const u32x4* xt = xs[t & 1];
        auto read_frag = [&](int f) {
            if constexpr (!LDSR) { return xconst[f % 4]; }
            const int row = (f % MB) * 16 + i16;
            return xt[row * CPR + swizzled_chunk_n<CPR>(row, 2 * g + f / MB)];
        };
        u32x4 ring[AHEAD + 1];
#pragma unroll
        for (int f = 0; f < AHEAD; f++) { ring[f] = read_frag(f); }
#pragma unroll
        for (int f = 0; f < FRAGS; f++)
        {
            if constexpr (GW && WL1) { if (f % WS == 0 && f / WS < NB) { load_w(f / WS); } }
            if (f == FRAGS / 2)
            {
                if constexpr (LDSW && !ST1)
                {
#pragma unroll
                    for (int i = 0; i < X_PER_THREAD; i++) { store_x(i); }
                }
                if constexpr (GX && !XL1)
                {
#pragma unroll
                    for (int i = 0; i < X_PER_THREAD; i++) { load_x(i); }
                }
            }
            if constexpr (LDSW && ST1) { if (f >= S0 && (f - S0) % SS == 0 && (f - S0) / SS < X_PER_THREAD) { store_x((f - S0) / SS); } }
            if constexpr (GX && XL1) { if (f >= S0 + 1 && (f - S0 - 1) % SS == 0 && (f - S0 - 1) / SS < X_PER_THREAD) { load_x((f - S0 - 1) / SS); } }
            if (f + AHEAD < FRAGS) { ring[(f + AHEAD) % (AHEAD + 1)] = read_frag(f + AHEAD); }
            const bf16x8 xf = __builtin_bit_cast(bf16x8, ring[f % (AHEAD + 1)]);
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
            {
                acc[f % MB][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wf[f / MB][nb]), xf, acc[f % MB][nb], 0, 0, 0);
            }
        }
        if constexpr (GW)
        {
#pragma unroll
            for (int nb = 0; nb < NB; nb++) { raw[nb] = rawn[nb]; }
        }
        if constexpr (LDSR)
        {
            // pin the order written above: the scheduler otherwise sinks every read to just before its use
            if constexpr (GW && !WL1) { __builtin_amdgcn_sched_group_barrier(0x020, NB, 0); }
            __builtin_amdgcn_sched_group_barrier(0x100, AHEAD, 0);
#pragma unroll
            for (int f = 0; f < FRAGS; f++)
            {
                if constexpr (GW && WL1) { if (f % WS == 0 && f / WS < NB) { __builtin_amdgcn_sched_group_barrier(0x020, 1, 0); } }
                if (f == FRAGS / 2)
                {
                    if constexpr (LDSW && !ST1) { __builtin_amdgcn_sched_group_barrier(0x200, X_PER_THREAD, 0); }
                    if constexpr (GX && !XL1) { __builtin_amdgcn_sched_group_barrier(0x020, X_PER_THREAD, 0); }
                }
                if constexpr (LDSW && ST1) { if (f >= S0 && (f - S0) % SS == 0 && (f - S0) / SS < X_PER_THREAD) { __builtin_amdgcn_sched_group_barrier(0x200, 1, 0); } }
                if constexpr (GX && XL1) { if (f >= S0 + 1 && (f - S0 - 1) % SS == 0 && (f - S0 - 1) / SS < X_PER_THREAD) { __builtin_amdgcn_sched_group_barrier(0x020, 1, 0); } }
                if (f + AHEAD < FRAGS) { __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); }
                __builtin_amdgcn_sched_group_barrier(0x008, NB, 0);
            }
        }
    }
    float total = 0.0f;
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++) { total += acc[mb][nb][0] + acc[mb][nb][1] + acc[mb][nb][2] + acc[mb][nb][3]; }
    if (total == -1.0f) { sink[0] = total + (float)xreg[0][0]; }           // keeps everything alive; never true for these operands
}

template <int FLAGS, int AHEAD = 3, int SCHED = 0, int WS = 1, int S0 = 8, int SS = 1>
__global__ __launch_bounds__(256, 2) void gemm_ablation_kernel(const int trips, const uint32_t seed, const uint8_t* __restrict__ wbuf,
                                                               const uint8_t* __restrict__ xbuf, float* __restrict__ sink)
{
    gemm_ablation_body<FLAGS, AHEAD, SCHED, WS, S0, SS>(trips, seed, wbuf, xbuf, sink);
}

template <int FLAGS, int AHEAD = 3, int SCHED = 0, int WS = 1, int S0 = 8, int SS = 1>
void launch_ablation(int wgs, int trips, uint32_t seed, const uint8_t* wbuf, const uint8_t* xbuf, float* sink)
{
    gemm_ablation_kernel<FLAGS, AHEAD, SCHED, WS, S0, SS><<<wgs, 256, 0, nullptr>>>(trips, seed, wbuf, xbuf, sink);
}

// the product kernel itself with a tile shape, k split and prefetch distance of the caller's choice
template <int MB, int NB, bool SPLIT, int PD, int WGS_PER_CU = 2>
void launch_product_kernel(const LinearArgs& a, int splits, float* partial)
{
    const int n_tiles = (a.n_out + 64 * NB - 1) / (64 * NB);
    const int m_tiles = (a.tokens + MB * 16 - 1) / (MB * 16);
    const dim3 grid(((n_tiles + 7) & ~7) * m_tiles, splits);
    gemm_mfma_direct_kernel<DT_E5M2, false, MB, SPLIT, true, DT_BF16, NB, false, false, PD, WGS_PER_CU><<<grid, 256, 0, nullptr>>>(a, n_tiles, SPLIT ? partial : nullptr);
    if (SPLIT) { launch_splitk_combine<DT_BF16>(partial, splits, a, nullptr); }
}

// tile 100 + 10 * shape + PD: shape 0 = 64 x 192, 1 = 64 x 256, 2 = 128 x 192, 3 = 64 x 256 split 4, 4 = 128 x 256 split 4,
// 5 = 64 x 256 split 2, 6 = 64 x 256 split 3, 7 = 128 x 192 split 2, 8 = 128 x 256 compiled for one workgroup per CU,
// 9 = the same split 4; PD 1 .. 3 (128-token tiles at two workgroups per CU: 1 or 2)
bool launch_product_tile(int tile, const LinearArgs& a, float* partial)
{
    switch (tile)
    {
    case 101: launch_product_kernel<4, 3, false, 1>(a, 1, partial); return true;
    case 102: launch_product_kernel<4, 3, false, 2>(a, 1, partial); return true;
    case 103: launch_product_kernel<4, 3, false, 3>(a, 1, partial); return true;
    case 111: launch_product_kernel<4, 4, false, 1>(a, 1, partial); return true;
    case 112: launch_product_kernel<4, 4, false, 2>(a, 1, partial); return true;
    case 113: launch_product_kernel<4, 4, false, 3>(a, 1, partial); return true;
    case 121: launch_product_kernel<8, 3, false, 1>(a, 1, partial); return true;
    case 122: launch_product_kernel<8, 3, false, 2>(a, 1, partial); return true;
    case 131: launch_product_kernel<4, 4, true, 1>(a, 4, partial); return true;
    case 132: launch_product_kernel<4, 4, true, 2>(a, 4, partial); return true;
    case 133: launch_product_kernel<4, 4, true, 3>(a, 4, partial); return true;
    case 141: launch_product_kernel<8, 4, true, 1>(a, 4, partial); return true;
    case 151: launch_product_kernel<4, 4, true, 1>(a, 2, partial); return true;
    case 153: launch_product_kernel<4, 4, true, 3>(a, 2, partial); return true;
    case 161: launch_product_kernel<4, 4, true, 1>(a, 3, partial); return true;
    case 163: launch_product_kernel<4, 4, true, 3>(a, 3, partial); return true;
    // 128 x 256 compiled for one workgroup per CU (512 registers per wave): unsplit and split in four
    case 181: launch_product_kernel<8, 4, false, 1, 1>(a, 1, partial); return true;
    case 182: launch_product_kernel<8, 4, false, 2, 1>(a, 1, partial); return true;
    case 183: launch_product_kernel<8, 4, false, 3, 1>(a, 1, partial); return true;
    case 191: launch_product_kernel<8, 4, true, 1, 1>(a, 4, partial); return true;
    case 192: launch_product_kernel<8, 4, true, 2, 1>(a, 4, partial); return true;
    case 193: launch_product_kernel<8, 4, true, 3, 1>(a, 4, partial); return true;
    case 201: launch_product_kernel<8, 2, true, 1>(a, 4, partial); return true;       // 128 x 128, k split in 4
    case 202: launch_product_kernel<8, 2, true, 2>(a, 4, partial); return true;
    case 211: launch_product_kernel<8, 2, false, 1>(a, 1, partial); return true;      // 128 x 128 unsplit
    case 171: launch_product_kernel<8, 3, true, 1>(a, 2, partial); return true;
    case 172: launch_product_kernel<8, 3, true, 2>(a, 2, partial); return true;
    default: return false;
    }
}

// the FP4 prefill kernel with its memory instructions in bursts (MEM_BURSTS) or one per token block
template <int MB, int NB, bool SPLIT, bool BURSTS>
void launch_fp4_kernel(const LinearArgs& a, const uint8_t* scales, int splits, float* partial)
{
    const int n_tiles = (a.n_out + 64 * NB - 1) / (64 * NB);
    const int m_tiles = (a.tokens + MB * 16 - 1) / (MB * 16);
    const dim3 grid(((n_tiles + 7) & ~7) * m_tiles, splits);
    gemm4_mfma_direct_kernel<16, MB, SPLIT, NB, false, false, BURSTS><<<grid, 256, 0, nullptr>>>(a, scales, n_tiles, SPLIT ? partial : nullptr);
    if (SPLIT) { launch_splitk_combine<DT_BF16>(partial, splits, a, nullptr); }
}

}    // namespace

extern "C" {

// Times `iters` launches of one variant on the tiled copies W_tiled[0 .. n_w) of E5M2 weights [n_out][K] (rotated),
// BF16 activations X [tokens][K], BF16 output Y [tokens][n_out] (n_out and tokens multiples of the tile).
// variant: bit 0 = SPREAD, bit 1 = RAST (4 x 2), bit 2 = TRACE; 16 / 17 / 18 = the memory instructions spread (three placements); 8 = the product entry (hip_quant_gemm, W_tiled then holds
// the row-major weights whose tiled copies are registered) in the same loop.  tile: see launch_tile.  inv_scale != 1: the scaled
// conversion (tile 0, no raster, no trace).  partial: tokens * n_out * 4 floats for tile 2.  Returns microseconds per
// launch (the combine launch of tile 2 included) or < 0; with TRACE, phases[0..3] receive the averages over all
// workgroups of the ticks spent converting (and waiting for weight bytes), at the barrier, in the rest of the k-tiles,
// and in the whole kernel.
// Microseconds per launch of gemm_ablation_kernel<flags>: 2 workgroups per CU, `trips` k-tiles per wave (each 64
// instructions of 16384 FLOPs), `launches` launches after two of warm-up.  flags: one of 0, 1, 3, 7, 15, 31, 63 (each adds
// one ingredient to the one before) or 2, 4, 16, 18 (single ingredients on the bare loop).
// FLOPs per launch = *n_workgroups * 4 * trips * 64 * 16384.
double cccc_bench_gemm_ablation(int flags, int trips, int launches, int* n_workgroups)
{
    if (trips <= 0 || launches <= 0 || !n_workgroups) { return -1.0; }
    hipDeviceProp_t prop;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) { return -1.0; }
    const int wgs = 2 * prop.multiProcessorCount;
    *n_workgroups = wgs;
    uint8_t* mem = nullptr;
    const size_t w_bytes = (size_t)16 * (256 << 10) + (1 << 20), x_bytes = (size_t)8 * (128 << 10) + (1 << 20);
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (hipMalloc(&mem, w_bytes + x_bytes + 256) != hipSuccess || hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) { return -3.0; }
    (void)hipMemset(mem, 0x3a, w_bytes + x_bytes + 256);          // finite FP8 codes and BF16 values
    float* sink = (float*)(mem + w_bytes + x_bytes);
    bool ok = true;
    for (int i = 0; i < launches + 2 && ok; i++)
    {
        if (i == 2) { (void)hipEventRecord(e0, nullptr); }
        const uint32_t seed = 0x12345u + i;
        switch (flags)
        {
        case 0: launch_ablation<0>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 1: launch_ablation<1>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 3: launch_ablation<3>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 7: launch_ablation<7>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 15: launch_ablation<15>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 31: launch_ablation<31>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 63: launch_ablation<63>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 2: launch_ablation<2>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 4: launch_ablation<4>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 16: launch_ablation<16>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 17: launch_ablation<17>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 6: launch_ablation<6>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        // the whole k-tile under other schedules: 1000 + 100 * AHEAD + SCHED
        case 1301: launch_ablation<63, 3, 1>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 1302: launch_ablation<63, 3, 2>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 1303: launch_ablation<63, 3, 3>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 1307: launch_ablation<63, 3, 7>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 1500: launch_ablation<63, 5, 0>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 1503: launch_ablation<63, 5, 3>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 1507: launch_ablation<63, 5, 7>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        // the product's order with other slots: weight loads every WS-th token block, stores from block S0 every SS-th
        case 4001: launch_ablation<63, 3, 7, 2, 8, 1>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 4002: launch_ablation<63, 3, 7, 4, 8, 1>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 4003: launch_ablation<63, 3, 7, 1, 4, 3>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 4004: launch_ablation<63, 3, 7, 1, 11, 1>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 4005: launch_ablation<63, 3, 7, 1, 2, 4>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 4006: launch_ablation<63, 3, 7, 4, 2, 4>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 4007: launch_ablation<63, 3, 7, 2, 7, 2>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 4008: launch_ablation<63, 3, 7, 1, 4, 1>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 1200: launch_ablation<63, 2, 0>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 2301: launch_ablation<15, 3, 1>(wgs, trips, seed, mem, mem + w_bytes, sink); break;      // up to the stores only
        case 2501: launch_ablation<15, 5, 1>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        case 2500: launch_ablation<15, 5, 0>(wgs, trips, seed, mem, mem + w_bytes, sink); break;
        default: ok = false; break;
        }
    }
    (void)hipEventRecord(e1, nullptr);
    double result = -2.0;
    if (ok && hipEventSynchronize(e1) == hipSuccess && hipGetLastError() == hipSuccess)
    {
        float ms = 0;
        (void)hipEventElapsedTime(&ms, e0, e1);
        result = (double)ms * 1000.0 / launches;
    }
    (void)hipDeviceSynchronize();
    (void)hipFree(mem);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return result;
}

// Times the FP4 (block 16) prefill kernel on the tiled copies W_tiled[0 .. n_w) (codes, then the scale bytes behind all
// code KiBs, as hip_quant_weight_prepare_fp4 writes them) of weights [n_out][K].  shape: 0 = 128 tokens x 256 features
// (one workgroup per CU), 1 = 64 x 256, 2 = 128 x 192, 3 = 128 x 256 with the k range split in `splits`.  bursts != 0: the
// memory instructions of a k-tile in two bursts instead of one per token block.  Microseconds per launch or < 0.
double cccc_bench_gemm4_variant(int shape, int bursts, int splits, int n_w, void** W_tiled, const void* X, void* Y, int n_out, int tokens, int K,
                                float* partial, int iters, int warmup)
{
    if (n_w <= 0 || !W_tiled || !X || !Y || iters <= 0 || K % 128 != 0 || tokens % 128 != 0 || n_out % (shape == 2 ? 192 : 256) != 0) { return -1.0; }
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) { return -1.0; }
    LinearArgs a{};
    a.X = (const uint16_t*)X;
    a.Y = (uint16_t*)Y;
    a.ldw = K;
    a.ldx = K;
    a.y_stride_tok = n_out;
    a.y_stride_out = 1;
    a.n_out = n_out;
    a.tokens = tokens;
    a.K = K;
    a.w_scale = 1.0f;
    a.alpha = 1.0f;
    a.beta = 0.0f;
    bool ok = true;
    for (int i = 0; i < warmup + iters && ok; i++)
    {
        if (i == warmup) { (void)hipEventRecord(e0, nullptr); }
        a.W = (const uint8_t*)W_tiled[i % n_w];
        const uint8_t* scales = a.W + (long long)((n_out + 15) / 16) * (K / 128) * 1024;
        switch (shape * 2 + (bursts ? 1 : 0))
        {
        case 0: launch_fp4_kernel<8, 4, false, false>(a, scales, 1, partial); break;
        case 1: launch_fp4_kernel<8, 4, false, true>(a, scales, 1, partial); break;
        case 2: launch_fp4_kernel<4, 4, false, false>(a, scales, 1, partial); break;
        case 3: launch_fp4_kernel<4, 4, false, true>(a, scales, 1, partial); break;
        case 4: launch_fp4_kernel<8, 3, false, false>(a, scales, 1, partial); break;
        case 5: launch_fp4_kernel<8, 3, false, true>(a, scales, 1, partial); break;
        case 6: launch_fp4_kernel<8, 4, true, false>(a, scales, splits, partial); break;
        case 7: launch_fp4_kernel<8, 4, true, true>(a, scales, splits, partial); break;
        default: ok = false; break;
        }
    }
    (void)hipEventRecord(e1, nullptr);
    double result = -2.0;
    if (ok && hipEventSynchronize(e1) == hipSuccess && hipGetLastError() == hipSuccess)
    {
        float ms = 0;
        (void)hipEventElapsedTime(&ms, e0, e1);
        result = (double)ms * 1000.0 / iters;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return result;
}

double cccc_bench_gemm_variant(int variant, int tile, int n_w, void** W_tiled, const void* X, void* Y, int n_out, int tokens, int K,
                               float inv_scale, float* partial, int iters, int warmup, double* phases)
{
    const bool wide3 = tile == 1 || tile == 4 || (tile >= 100 && (tile / 10 == 10 || tile / 10 == 12 || tile / 10 == 17));
    const bool narrow = tile >= 200;           // 128-feature tiles
    if (n_w <= 0 || !W_tiled || !X || !Y || iters <= 0 || K % 64 != 0 || tokens % 128 != 0 || n_out % (wide3 ? 192 : (narrow ? 128 : 256)) != 0) { return -1.0; }
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) { return -1.0; }
    unsigned long long* trace = nullptr;
    const size_t trace_slots = 16384;
    if ((variant & 4) && hipMalloc(&trace, trace_slots * 4 * sizeof(unsigned long long)) != hipSuccess) { return -3.0; }
    if (trace) { (void)hipMemset(trace, 0, trace_slots * 4 * sizeof(unsigned long long)); }
    LinearArgs a{};
    a.X = (const uint16_t*)X;
    a.Y = (uint16_t*)Y;
    a.ldw = K;
    a.ldx = K;
    a.y_stride_tok = n_out;
    a.y_stride_out = 1;
    a.n_out = n_out;
    a.tokens = tokens;
    a.K = K;
    a.w_scale = inv_scale;
    a.alpha = 1.0f;
    a.beta = 0.0f;
    unsigned n_wgs = 0;
    bool ok = true;
    const int previous_sync = hip_quant_set_sync(0);
    for (int i = 0; i < warmup + iters && ok; i++)
    {
        if (i == warmup) { (void)hipEventRecord(e0, nullptr); }
        a.W = (const uint8_t*)W_tiled[i % n_w];
        const bool scaled = inv_scale != 1.0f;
        if (tile >= 100)
        {
            ok = variant == 0 && !scaled && launch_product_tile(tile, a, partial);
            continue;
        }
        switch (variant)
        {
        case 0: ok = launch_tile<false, false, false>(tile, scaled, a, partial, trace, &n_wgs); break;
        case 1: ok = launch_tile<true, false, false>(tile, scaled, a, partial, trace, &n_wgs); break;
        case 2: ok = launch_tile<false, true, false>(tile, scaled, a, partial, trace, &n_wgs); break;
        case 3: ok = launch_tile<true, true, false>(tile, scaled, a, partial, trace, &n_wgs); break;
        case 4: ok = launch_tile<false, false, true>(tile, scaled, a, partial, trace, &n_wgs); break;
        case 5: ok = launch_tile<true, false, true>(tile, scaled, a, partial, trace, &n_wgs); break;
        case 16: ok = !scaled && launch_tile_memspread<1>(tile, a, partial, &n_wgs); break;
        case 17: ok = !scaled && launch_tile_memspread<2>(tile, a, partial, &n_wgs); break;
        case 18: ok = !scaled && launch_tile_memspread<3>(tile, a, partial, &n_wgs); break;
        case 8:
            ok = hip_quant_gemm(1, 0, n_out, tokens, K, 1.0f, a.W, (int)DT_E5M2, K, inv_scale, X, (int)DT_BF16, K, 1.0f, 0.0f, Y, (int)DT_BF16, n_out, 0.0f,
                                nullptr, nullptr, 0) == 0;
            break;
        default: ok = false; break;
        }
    }
    (void)hipEventRecord(e1, nullptr);
    hip_quant_set_sync(previous_sync);
    double result = -2.0;
    if (ok && hipEventSynchronize(e1) == hipSuccess && hipGetLastError() == hipSuccess)
    {
        float ms = 0;
        (void)hipEventElapsedTime(&ms, e0, e1);
        result = (double)ms * 1000.0 / iters;
    }
    if (trace && phases && result > 0 && n_wgs <= trace_slots)
    {
        unsigned long long* h = new unsigned long long[(size_t)n_wgs * 4];
        if (hipMemcpy(h, trace, (size_t)n_wgs * 4 * sizeof(unsigned long long), hipMemcpyDeviceToHost) == hipSuccess)
        {
            double s[4] = { 0, 0, 0, 0 };
            unsigned n = 0;
            for (unsigned w = 0; w < n_wgs; w++)
            {
                if (h[w * 4 + 3] == 0) { continue; }          // a padding workgroup
                for (int j = 0; j < 4; j++) { s[j] += (double)h[w * 4 + j]; }
                n++;
            }
            for (int j = 0; j < 4; j++) { phases[j] = n ? s[j] / n : 0.0; }
        }
        delete[] h;
    }
    if (trace) { (void)hipFree(trace); }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return result;
}

}    // extern "C"
