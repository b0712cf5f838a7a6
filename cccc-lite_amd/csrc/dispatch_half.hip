#include "dispatch_half.h"
#include "gemm_kernels.h"
#include "gemv_dispatch.h"
#include "gemv_kernels.h"
#include "runtime.h"

namespace ccq
{

namespace
{

template <int WT, int MT, int R, int WAVES, int OCC, bool SCALED>
void launch_half_gemv(const LinearArgs& a)
{
    const int n_groups = (a.n_out + R - 1) / R;
    const int want = (n_groups + WAVES - 1) / WAVES;
    const int cap = cu_count() * OCC;
    const size_t lds = (size_t)MT * ((a.K + 1023) / 1024) * 2048;
    gemv8_dot2_kernel<WT, MT, R, 4, WAVES, SCALED, DT_HALF><<<want < cap ? want : cap, WAVES * 64, lds, stream()>>>(a);
}

// the two shapes of the BF16 dispatch that matter most: tall weights and long rows take 8-wave workgroups
template <int WT, int MT, bool SCALED>
void pick_half_gemv(const LinearArgs& a)
{
    if (a.K > 8192 || a.n_out / cu_count() >= 128) { launch_half_gemv<WT, MT, 1, 8, 2, SCALED>(a); }
    else { launch_half_gemv<WT, MT, 2, 4, 4, SCALED>(a); }
}

template <int WT, bool SCALED>
bool half_gemv(const LinearArgs& a)
{
    if ((size_t)a.tokens * ((a.K + 1023) / 1024) * 2048 > 64 * 1024) { return false; }
    switch (a.tokens)
    {
    case 1: pick_half_gemv<WT, 1, SCALED>(a); return true;
    case 2: pick_half_gemv<WT, 2, SCALED>(a); return true;
    case 3: pick_half_gemv<WT, 3, SCALED>(a); return true;
    case 4: pick_half_gemv<WT, 4, SCALED>(a); return true;
    default: return false;
    }
}


template <int WT>
bool half_mfma_gemv(const LinearArgs& a, const uint8_t* tiled)
{
    const bool scaled = a.w_scale != 1.0f;
    if (tiled) { return scaled ? gemv8_mfma_ksplit_tiled<WT, true, DT_HALF>(a, tiled) : gemv8_mfma_ksplit_tiled<WT, false, DT_HALF>(a, tiled); }
    return scaled ? gemv8_mfma<WT, true, DT_HALF>(a) : gemv8_mfma<WT, false, DT_HALF>(a);
}

}    // namespace

// Kernel choice as for BF16 activations (dispatch.hip): with a tiled copy the matrix-core GEMV on it for up to 16 tokens
// (one or two tokens of a weight under 8 MiB stay on the dot2 kernel), else dot2 up to 4 tokens and the matrix-core GEMV
// on the row-major bytes up to 16 (4096 x 12288 at 16 tokens: 16.3 us on the GEMM kernel this replaced there), the GEMM above.
const char* half_linear(const LinearArgs& a, int w_type, SplitScratch* scratch)
{
    const bool scaled = a.w_scale != 1.0f;
    const uint8_t* tiled = lookup_tiled(a.W, w_type, a.n_out, a.K, a.ldw);
    if (tiled && a.tokens <= 16 && (a.tokens >= 3 || (long long)a.n_out * a.K >= (8LL << 20)))
    {
        if (w_type == DT_E5M2 ? half_mfma_gemv<DT_E5M2>(a, tiled) : half_mfma_gemv<DT_E4M3>(a, tiled)) { return "gemv_mfma_tiled_half"; }
    }
    if (a.tokens <= 4)
    {
        bool ok;
        if (w_type == DT_E5M2) { ok = scaled ? half_gemv<DT_E5M2, true>(a) : half_gemv<DT_E5M2, false>(a); }
        else { ok = scaled ? half_gemv<DT_E4M3, true>(a) : half_gemv<DT_E4M3, false>(a); }
        if (ok) { return "gemv_dot2_half"; }
    }
    if (a.tokens <= 16)
    {
        if (w_type == DT_E5M2 ? half_mfma_gemv<DT_E5M2>(a, nullptr) : half_mfma_gemv<DT_E4M3>(a, nullptr)) { return "gemv_mfma_half"; }
    }
    const bool launched = w_type == DT_E5M2 ? gemm_mfma<DT_E5M2, 0, DT_HALF>(a, tiled, scratch) : gemm_mfma<DT_E4M3, 0, DT_HALF>(a, tiled, scratch);
    return launched ? "gemm_mfma_half" : nullptr;
}

}    // namespace ccq
