// Launch choice of the matrix-core GEMV (gemv8_mfma_kernel, 1..16 tokens), shared by the BF16 and the HALF dispatcher.
// The shapes were tuned on MI355X over the Qwen3-8B weights with rotating buffers (no cache reuse); they live in one
// table so that another shape family only adds rows.
#pragma once
#include "gemv_kernels.h"
#include "runtime.h"
#include <climits>

namespace ccq
{

// One configuration of the kernel on the tiled copy: RT row tiles (16 rows each) per workgroup, U k-blocks of 64 in flight
// per wave and trip, WAVES waves that split K between them, XLDS = activations through a wave-private LDS slab.
struct TiledGemvConfig
{
    int rt, u, waves;
    bool xlds;
};

// A row applies when the weight's row tiles per compute unit, its K and the token count fall inside the row's ranges (and,
// where `three_halves` is set, when there are at least 1.5 row tiles per compute unit); the first row that applies is taken.
struct TiledGemvRule
{
    int min_tiles_per_cu, max_tiles_per_cu;
    int min_K, max_K;
    int max_tokens;
    bool three_halves;
    TiledGemvConfig config;
};

// From five tokens on the activation operand goes through LDS (XLDS, see the kernel): fetched in operand order it costs 16
// cache lines per 256 bytes, and at 16 tokens that, not HBM, bounds the kernel (K = 12288, 4096 rows: 15.2 -> 13.3 us;
// K = 4096, 1024 rows: 6.4 -> 5.3 us).
constexpr TiledGemvRule kTiledGemvRules[] = {
    //  tiles / CU      K                 tokens  >= 1.5 tiles / CU   RT  U  waves  XLDS
    // tall weights (lm_head, gate + up stored together): several row tiles per workgroup
    { 16, INT_MAX,      0, INT_MAX,       4,      false,              { 2, 2, 8, false } },
    { 16, INT_MAX,      0, INT_MAX,       8,      false,              { 2, 2, 8, true } },
    { 16, INT_MAX,      0, INT_MAX,       16,     false,              { 4, 2, 8, true } },
    // projections stored together (gate + up: 24576 rows, q + k + v: 6144 rows), one or two tokens
    { 4, 15,            0, INT_MAX,       2,      false,              { 2, 2, 16, false } },
    { 0, 1,             0, 8192,          2,      true,               { 2, 4, 8, false } },
    // 2 .. 15 row tiles per compute unit (4096 x 12288)
    { 2, 15,            0, INT_MAX,       2,      false,              { 1, 1, 8, false } },
    { 2, 15,            0, INT_MAX,       4,      false,              { 2, 1, 8, false } },
    { 2, 15,            0, INT_MAX,       8,      false,              { 1, 1, 8, true } },
    { 2, 15,            0, INT_MAX,       16,     false,              { 4, 2, 8, true } },
    // few row tiles, long rows (12288 x 4096): one tile per workgroup, K split over the waves
    { 0, 1,             8193, INT_MAX,    4,      false,              { 1, 4, 8, false } },
    { 0, 1,             8193, INT_MAX,    8,      false,              { 1, 2, 16, true } },
    { 0, 1,             8193, INT_MAX,    16,     false,              { 1, 4, 8, true } },
    // few row tiles, short rows (4096 x 4096, 4096 x 1024)
    { 0, 1,             0, 8192,          4,      false,              { 1, 2, 16, false } },
    { 0, 1,             0, 8192,          8,      false,              { 1, 2, 16, true } },
    { 0, 1,             0, 8192,          16,     false,              { 1, 4, 8, true } },
};

inline TiledGemvConfig pick_tiled_gemv(int n_out, int K, int tokens)
{
    const int cus = cu_count();
    const int n_tiles = (n_out + 15) / 16;
    const int per_cu = n_tiles / cus;
    for (const TiledGemvRule& r : kTiledGemvRules)
    {
        if (per_cu < r.min_tiles_per_cu || per_cu > r.max_tiles_per_cu || K < r.min_K || K > r.max_K || tokens > r.max_tokens) { continue; }
        if (r.three_halves && 2 * n_tiles < 3 * cus) { continue; }
        return r.config;
    }
    return TiledGemvConfig{ 1, 4, 8, true };
}

template <int WT, int RT, int U, int WAVES, bool SCALED, bool XLDS, int AT>
void launch_tiled_gemv(const LinearArgs& t)
{
    gemv8_mfma_kernel<WT, RT, U, WAVES, SCALED, true, XLDS, AT><<<(t.n_out + 16 * RT - 1) / (16 * RT), WAVES * 64, 0, stream()>>>(t);
}

// The matrix-core GEMV on the load-time tiled copy `tiled` of a.W: every load instruction of a wave covers one contiguous
// KiB and a workgroup walks one contiguous row tile, which streams better than the row-major kernels at every token count
// (lm_head, one token: 89.8 us against 92.7 for the dot2 kernel).  False: the table names a configuration that is not
// instantiated (nothing launched).
template <int WT, bool SCALED, int AT = DT_BF16>
bool gemv8_mfma_ksplit_tiled(const LinearArgs& a, const uint8_t* tiled)
{
    LinearArgs t = a;
    t.W = tiled;
    const TiledGemvConfig c = pick_tiled_gemv(a.n_out, a.K, a.tokens);
    const int key = c.rt * 1000 + c.u * 100 + c.waves;
    if (!c.xlds)
    {
        switch (key)
        {
        case 2208: launch_tiled_gemv<WT, 2, 2, 8, SCALED, false, AT>(t); return true;
        case 2216: launch_tiled_gemv<WT, 2, 2, 16, SCALED, false, AT>(t); return true;
        case 2408: launch_tiled_gemv<WT, 2, 4, 8, SCALED, false, AT>(t); return true;
        case 1108: launch_tiled_gemv<WT, 1, 1, 8, SCALED, false, AT>(t); return true;
        case 2108: launch_tiled_gemv<WT, 2, 1, 8, SCALED, false, AT>(t); return true;
        case 1408: launch_tiled_gemv<WT, 1, 4, 8, SCALED, false, AT>(t); return true;
        case 1216: launch_tiled_gemv<WT, 1, 2, 16, SCALED, false, AT>(t); return true;
        default: return false;
        }
    }
    switch (key)
    {
    case 2208: launch_tiled_gemv<WT, 2, 2, 8, SCALED, true, AT>(t); return true;
    case 4208: launch_tiled_gemv<WT, 4, 2, 8, SCALED, true, AT>(t); return true;
    case 1108: launch_tiled_gemv<WT, 1, 1, 8, SCALED, true, AT>(t); return true;
    case 1216: launch_tiled_gemv<WT, 1, 2, 16, SCALED, true, AT>(t); return true;
    case 1408: launch_tiled_gemv<WT, 1, 4, 8, SCALED, true, AT>(t); return true;
    default: return false;
    }
}

// The same kernel on the row-major bytes, 5..16 tokens: activations through LDS as on the tiled copy.
template <int WT, bool SCALED, int AT = DT_BF16>
bool gemv8_mfma(const LinearArgs& a)
{
    if (a.n_out >= cu_count() * 32) { gemv8_mfma_kernel<WT, 4, 2, 4, SCALED, false, true, AT><<<(a.n_out + 63) / 64, 256, 0, stream()>>>(a); }
    else { gemv8_mfma_kernel<WT, 1, 2, 8, SCALED, false, true, AT><<<(a.n_out + 15) / 16, 512, 0, stream()>>>(a); }
    return true;
}

}    // namespace ccq
