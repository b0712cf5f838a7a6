// hip_quant_gemm: the unified quantized GEMM entry point.  Normalises the BLAS-style arguments of
// the reference's dispatcher (cccc/cublas_real.h:875-880) into "one quantized linear" and picks a
// kernel family by token count:
//     tokens <= 4   gemv_dot2   (FP8 / FP4, dot2 + DPP)
//     tokens <= 16  gemv_mfma   (FP8), token groups of 4 through gemv_dot2 (FP4)
//     otherwise     gemm_mfma   (dequant-to-LDS + bf16 MFMA)
//     anything the fast kernels cannot take (transposed layouts, odd sizes, misaligned pointers,
//     FP4 without block scales): generic
#include "../../include/cccc_hip_quant.h"
#include "gemv_kernels.h"
#include "gemm_kernels.h"
#include "runtime.h"
#include <cstdio>

using namespace ccq;

namespace
{

inline bool is_quantized(int t) { return t == DT_E4M3 || t == DT_E5M2 || t == DT_FP4; }
inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

constexpr int kMaxLds = 160 * 1024;

// Raises a kernel's dynamic LDS limit once; returns false if the runtime refuses.
template <typename Kernel>
bool allow_big_lds(Kernel kernel, size_t bytes)
{
    if (bytes <= 64 * 1024) { return true; }
    if (bytes > (size_t)kMaxLds) { return false; }
    static thread_local Kernel done_for = nullptr;
    if (done_for == kernel) { return true; }
    if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds) != hipSuccess)
    {
        (void)hipGetLastError();
        return false;
    }
    done_for = kernel;
    return true;
}

// One FP8 GEMV launch: PIPE picks the software-pipelined variant, OCC workgroups per CU cap the grid
// (the kernels walk the row groups with a grid stride).
template <int WT, int MT, int R, int U, int WAVES, int OCC, bool PIPE, bool SCALED>
bool launch_gemv8_dot2(const LinearArgs& a)
{
    const size_t lds = (size_t)MT * ((a.K + 1023) / 1024) * 2048;
    auto kernel = PIPE ? gemv8_dot2_pipe_kernel<WT, MT, R, U, WAVES, SCALED, true> : gemv8_dot2_kernel<WT, MT, R, U, WAVES, SCALED>;
    if (!allow_big_lds(kernel, lds)) { return false; }
    const int n_groups = (a.n_out + R - 1) / R;
    const int want = (n_groups + WAVES - 1) / WAVES;
    const int cap = cu_count() * (lds > 80 * 1024 ? 1 : (lds > 40 * 1024 && OCC > 2 ? 2 : OCC));
    kernel<<<want < cap ? want : cap, WAVES * 64, lds, stream()>>>(a);
    return true;
}

// Shapes were tuned on MI355X with rotating weight buffers (no cache reuse): small weights want
// every row in flight at once (one row per wave, pipelined), mid-size ones two rows per wave,
// very tall ones (lm_head) one row per wave again with more waves per workgroup.
template <int WT, int MT, bool SCALED>
bool pick_gemv8_dot2(const LinearArgs& a)
{
    const long long bytes = (long long)a.n_out * a.K;
    const long long rows_per_cu = a.n_out / cu_count();
    if (MT <= 2)
    {
        if (bytes <= (8LL << 20)) { return launch_gemv8_dot2<WT, MT, 1, 4, 8, 2, true, SCALED>(a); }
        if (rows_per_cu >= 128) { return launch_gemv8_dot2<WT, MT, 1, 4, 8, 2, false, SCALED>(a); }
        if (a.K > 8192) { return launch_gemv8_dot2<WT, MT, 2, 4, 8, 2, false, SCALED>(a); }
        return launch_gemv8_dot2<WT, MT, 2, 4, 4, 4, false, SCALED>(a);
    }
    if (rows_per_cu >= 128) { return launch_gemv8_dot2<WT, MT, 2, 4, 4, 4, false, SCALED>(a); }
    return launch_gemv8_dot2<WT, MT, 1, 4, 16, 1, false, SCALED>(a);
}

template <int WT, bool SCALED>
bool gemv8_dot2(const LinearArgs& a)
{
    switch (a.tokens)
    {
    case 1: return pick_gemv8_dot2<WT, 1, SCALED>(a);
    case 2: return pick_gemv8_dot2<WT, 2, SCALED>(a);
    case 3: return pick_gemv8_dot2<WT, 3, SCALED>(a);
    case 4: return pick_gemv8_dot2<WT, 4, SCALED>(a);
    default: return false;
    }
}

template <int WT, bool SCALED>
bool gemv8_mfma(const LinearArgs& a)
{
    const int cus = cu_count();
    if (a.n_out >= cus * 32) { gemv8_mfma_kernel<WT, 4, 2, 4, SCALED><<<(a.n_out + 63) / 64, 256, 0, stream()>>>(a); }
    else { gemv8_mfma_kernel<WT, 1, 2, 8, SCALED><<<(a.n_out + 15) / 16, 512, 0, stream()>>>(a); }
    return true;
}

template <int MT, int BLOCK>
bool launch_gemv4_dot2(const LinearArgs& a)
{
    const size_t lds = (size_t)MT * ((a.K + 2047) / 2048) * 4096;
    const long long rows_per_cu = a.n_out / cu_count();
    if (rows_per_cu >= 32)
    {
        auto kernel = gemv4_dot2_kernel<MT, 2, 2, 4, BLOCK>;
        if (!allow_big_lds(kernel, lds)) { return false; }
        const int want = ((a.n_out + 1) / 2 + 3) / 4;
        const int cap = cu_count() * (lds > 80 * 1024 ? 1 : 4);
        kernel<<<want < cap ? want : cap, 256, lds, stream()>>>(a);
    }
    else
    {
        auto kernel = gemv4_dot2_kernel<MT, 1, 2, 4, BLOCK>;
        if (!allow_big_lds(kernel, lds)) { return false; }
        const int want = (a.n_out + 3) / 4;
        const int cap = cu_count() * (lds > 80 * 1024 ? 1 : 4);
        kernel<<<want < cap ? want : cap, 256, lds, stream()>>>(a);
    }
    return true;
}

template <int BLOCK>
bool gemv4_dot2(const LinearArgs& a)
{
    switch (a.tokens)
    {
    case 1: return launch_gemv4_dot2<1, BLOCK>(a);
    case 2: return launch_gemv4_dot2<2, BLOCK>(a);
    case 3: return launch_gemv4_dot2<3, BLOCK>(a);
    case 4: return launch_gemv4_dot2<4, BLOCK>(a);
    default: return false;
    }
}

void launch_generic(const GenericArgs& g)
{
    const long long total = (long long)g.n_out * g.tokens;
    long long blocks = (total + 255) / 256;
    const long long cap = (long long)cu_count() * 32;
    if (blocks > cap) { blocks = cap; }
    if (blocks < 1) { blocks = 1; }
    generic_linear_kernel<<<(unsigned)blocks, 256, 0, stream()>>>(g);
}

}    // namespace

int hip_quant_gemm(int transA, int transB, int M, int N, int K, float alpha,
                   const void* A, int typeA, int lda, float invScaleA,
                   const void* B, int typeB, int ldb, float invScaleB,
                   float beta, void* C, int typeC, int ldc, float /*act_scale*/,
                   const void* blk_scA, const void* blk_scB, unsigned int block_size)
{
    const bool aQ = is_quantized(typeA), bQ = is_quantized(typeB);
    if (aQ == bQ || typeC != DT_BF16) { return -1; }
    if ((aQ && typeB != DT_BF16) || (bQ && typeA != DT_BF16)) { return -1; }
    if ((transA != 0 && transA != 1) || (transB != 0 && transB != 1)) { return -1; }
    if (M < 0 || N < 0 || K < 0 || lda <= 0 || ldb <= 0 || ldc <= 0) { return -1; }
    if (M == 0 || N == 0) { return 0; }
    if (!A || !B || !C) { return -1; }

    GenericArgs g{};
    g.K = K;
    g.alpha = alpha;
    g.beta = beta;
    g.Y = (uint16_t*)C;
    if (aQ)
    {
        g.W = (const uint8_t*)A;
        g.w_type = typeA;
        g.w_scale = invScaleA;
        g.blk_sc = (typeA == DT_FP4) ? (const uint8_t*)blk_scA : nullptr;
        g.w_stride_out = transA ? lda : 1;
        g.w_stride_k = transA ? 1 : lda;
        g.X = (const uint16_t*)B;
        g.x_stride_tok = transB ? 1 : ldb;
        g.x_stride_k = transB ? ldb : 1;
        g.n_out = M;
        g.tokens = N;
        g.y_stride_out = 1;
        g.y_stride_tok = ldc;
    }
    else
    {
        g.W = (const uint8_t*)B;
        g.w_type = typeB;
        g.w_scale = invScaleB;
        g.blk_sc = (typeB == DT_FP4) ? (const uint8_t*)blk_scB : nullptr;
        g.w_stride_out = transB ? 1 : ldb;
        g.w_stride_k = transB ? ldb : 1;
        g.X = (const uint16_t*)A;
        g.x_stride_tok = transA ? lda : 1;
        g.x_stride_k = transA ? 1 : lda;
        g.n_out = N;
        g.tokens = M;
        g.y_stride_out = ldc;
        g.y_stride_tok = 1;
    }
    g.block_size = block_size ? block_size : 16;
    if (g.blk_sc) { g.w_scale = 1.0f; }

    bool launched = false;
    const bool k_major = g.w_stride_k == 1 && g.x_stride_k == 1 && K > 0;
    if (k_major)
    {
        LinearArgs a{};
        a.W = g.W;
        a.blk_sc = g.blk_sc;
        a.X = g.X;
        a.Y = g.Y;
        a.ldw = g.w_stride_out;
        a.ldx = g.x_stride_tok;
        a.y_stride_tok = g.y_stride_tok;
        a.y_stride_out = g.y_stride_out;
        a.n_out = g.n_out;
        a.tokens = g.tokens;
        a.K = K;
        a.block_size = g.block_size;
        a.w_scale = g.w_scale;
        a.alpha = alpha;
        a.beta = beta;
        const bool x_ok = aligned16(a.X) && a.ldx % 8 == 0;
        if (g.w_type == DT_FP4)
        {
            const bool ok = x_ok && a.blk_sc && (a.block_size == 16 || a.block_size == 32) && K % 32 == 0 && a.ldw % 32 == 0 &&
                            aligned16(a.W) && ((uintptr_t)a.blk_sc & 1u) == 0;
            if (ok && a.tokens <= 16)
            {
                // token groups of up to four share one pass over the weight
                launched = true;
                for (int t0 = 0; t0 < g.tokens && launched; t0 += 4)
                {
                    LinearArgs s = a;
                    s.tokens = (g.tokens - t0 < 4) ? g.tokens - t0 : 4;
                    s.X = a.X + (long long)t0 * a.ldx;
                    s.Y = a.Y + (long long)t0 * a.y_stride_tok;
                    launched = a.block_size == 16 ? gemv4_dot2<16>(s) : gemv4_dot2<32>(s);
                }
                if (launched) { note_kernel("gemv_dot2"); }
            }
            else if (ok)
            {
                launched = a.block_size == 16 ? gemm_mfma<DT_FP4, 16>(a) : gemm_mfma<DT_FP4, 32>(a);
                if (launched) { note_kernel("gemm_mfma"); }
            }
        }
        else
        {
            const bool ok = x_ok && K % 16 == 0 && a.ldw % 16 == 0 && aligned16(a.W);
            const bool scaled = a.w_scale != 1.0f;
            if (ok && a.tokens <= 4)
            {
                if (g.w_type == DT_E5M2) { launched = scaled ? gemv8_dot2<DT_E5M2, true>(a) : gemv8_dot2<DT_E5M2, false>(a); }
                else { launched = scaled ? gemv8_dot2<DT_E4M3, true>(a) : gemv8_dot2<DT_E4M3, false>(a); }
                if (launched) { note_kernel("gemv_dot2"); }
            }
            if (ok && !launched && a.tokens <= 16)
            {
                if (g.w_type == DT_E5M2) { launched = scaled ? gemv8_mfma<DT_E5M2, true>(a) : gemv8_mfma<DT_E5M2, false>(a); }
                else { launched = scaled ? gemv8_mfma<DT_E4M3, true>(a) : gemv8_mfma<DT_E4M3, false>(a); }
                if (launched) { note_kernel("gemv_mfma"); }
            }
            if (ok && !launched)
            {
                if (g.w_type == DT_E5M2) { launched = gemm_mfma<DT_E5M2, 0>(a); }
                else { launched = gemm_mfma<DT_E4M3, 0>(a); }
                if (launched) { note_kernel("gemm_mfma"); }
            }
        }
    }
    if (!launched)
    {
        launch_generic(g);
        note_kernel("generic");
    }
    return finish("quant_gemm");
}
