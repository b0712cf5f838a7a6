// hip_quant_gemm: the unified quantized GEMM entry point.  Normalises the BLAS-style arguments of
// the reference's dispatcher (cccc/cublas_real.h:875-880) into "one quantized linear" and picks a
// kernel family:
//     FP8, tokens <= 16, tiled copy registered     gemv_mfma_tiled (matrix cores over the load-time copy; one or
//                                                  two tokens on a weight under 8 MiB stay on gemv_dot2)
//     FP8, tokens <= 4                             gemv_dot2 (dot2 + DPP, software pipelined for small weights)
//     FP8, tokens 5..16                            gemv_mfma (matrix cores, row-major weight)
//     FP8, tokens >= 17                            gemm_mfma: weights straight into the matrix-core operands when
//                                                  tokens >= 17 and K % 64 == 0 (row-major or tiled copy, k split
//                                                  over workgroups when the output has few tiles), else dequant-to-LDS
//     FP4 block scales, tiled copy registered      tokens <= 16: gemv_mfma_tiled (matrix cores, one pass over the weight for
//                                                  up to 16 tokens; one or two tokens of a short row stay on gemv_dot2);
//                                                  tokens >= 17 and K % 128 == 0: gemm_mfma_tiled (codes and scales straight
//                                                  into the matrix-core operands, k split when the output has few tiles)
//     FP4 block scales, no tiled copy              gemv_dot2 in token groups of four; tokens >= 17: gemm_mfma (dequant-to-LDS)
//     HALF activations                             the half instantiations of gemv_dot2 / gemm_mfma
//     anything the fast kernels cannot take (transposed layouts, odd sizes, misaligned pointers,
//     FP4 without block scales): generic
// Also here, for a prompt's T tokens on the register-fed GEMM kernels: hip_quant_gemm_segments (q, k, v in one launch),
// hip_quant_gemm_swiglu (gate, up and their SwiGLU product) and hip_quant_gemm_add_rms_norm (a k-split linear whose combine
// launch adds the residual and norms the row).
#include "../../include/cccc_hip_quant.h"
#include "gemv_kernels.h"
#include "gemv_dispatch.h"
#include "dispatch_half.h"
#include "gemm_kernels.h"
#include "runtime.h"
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <shared_mutex>
#include <unordered_map>
#include <unordered_set>

// Scratch of hip_quant_gemm_noalloc: the FP32 partial sums of a k-split GEMM.  One copy per GPU the library
// runs on, held until the process ends; every call on a GPU shares it.
static __device__ __align__(256) unsigned char scratch[HIP_QUANT_NOALLOC_SCRATCH_BYTES];

using namespace ccq;

namespace
{

inline bool is_quantized(int t) { return t == DT_E4M3 || t == DT_E5M2 || t == DT_FP4; }
inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

constexpr int kMaxLds = 160 * 1024;

// Raises a kernel's dynamic LDS limit the first time it is needed; returns false if the runtime refuses.
template <typename Kernel>
bool allow_big_lds(Kernel kernel, size_t bytes)
{
    if (bytes <= 64 * 1024) { return true; }
    if (bytes > (size_t)kMaxLds) { return false; }
    static std::mutex mutex;
    static std::unordered_set<const void*> raised;
    std::lock_guard<std::mutex> lock(mutex);
    if (raised.count((const void*)kernel)) { return true; }
    if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds) != hipSuccess)
    {
        (void)hipGetLastError();
        return false;
    }
    raised.insert((const void*)kernel);
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

// ---- load-time repacked weights: caller's weight pointer -> tiled copy
struct TiledWeight
{
    const uint8_t* tiled;
    int type, n_out, K;
    long long ldw;
    const void* blk_sc;      // FP4: the block scales the copy was built from, and their block length
    unsigned block;
};
std::shared_mutex g_tiled_mutex;
std::unordered_map<const void*, TiledWeight> g_tiled;

const uint8_t* find_tiled(const LinearArgs& a, int type) { return ccq::lookup_tiled(a.W, type, a.n_out, a.K, a.ldw); }

// block length the FP4 tiled copy registered under W was built with (0: none)
unsigned tiled_block_of(const void* W)
{
    std::shared_lock<std::shared_mutex> lock(g_tiled_mutex);
    const auto it = g_tiled.find(W);
    return it == g_tiled.end() ? 0u : it->second.block;
}

// The tiled copy of an FP4 weight, if one was built from these codes, these block scales and this block length.
const uint8_t* find_tiled_fp4(const LinearArgs& a)
{
    std::shared_lock<std::shared_mutex> lock(g_tiled_mutex);
    if (g_tiled.empty()) { return nullptr; }
    const auto it = g_tiled.find(a.W);
    if (it == g_tiled.end()) { return nullptr; }
    const TiledWeight& t = it->second;
    return (t.type == DT_FP4 && t.n_out == a.n_out && t.K == a.K && t.ldw == a.ldw && t.blk_sc == a.blk_sc && t.block == a.block_size) ? t.tiled : nullptr;
}

// FP4 on the matrix cores over the tiled copy.  Launch shapes follow the FP8 kernel's (one row tile per workgroup
// while tiles are scarce, K split over 8 or 16 waves); four-token and sixteen-token instantiations.
template <int BLOCK, int RT, int U, int WAVES>
void launch_gemv4_mfma(const LinearArgs& t, const uint8_t* scales)
{
    const unsigned grid = (t.n_out + 16 * RT - 1) / (16 * RT);
    if (t.tokens <= 4) { gemv4_mfma_kernel<BLOCK, RT, U, WAVES, 4><<<grid, WAVES * 64, 0, stream()>>>(t, scales); }
    else { gemv4_mfma_kernel<BLOCK, RT, U, WAVES, 16><<<grid, WAVES * 64, 0, stream()>>>(t, scales); }
}

template <int BLOCK>
bool gemv4_mfma_tiled(const LinearArgs& a, const uint8_t* tiled)
{
    LinearArgs t = a;
    t.W = tiled;
    const int n_tiles = (a.n_out + 15) / 16;
    const uint8_t* scales = tiled + (long long)n_tiles * ((a.K + 127) / 128) * 1024;
    // tuned on MI355X over the Llama-3.1-8B shapes with rotating weights; the kernel is bound by its conversion and
    // scaling arithmetic more than by bytes, so few-tile shapes want as many waves as a workgroup can hold
    const int tiles_per_cu = n_tiles / cu_count();
    if (tiles_per_cu >= 16)
    {
        if (a.tokens <= 8) { launch_gemv4_mfma<BLOCK, 2, 1, 8>(t, scales); }
        else { launch_gemv4_mfma<BLOCK, 4, 1, 8>(t, scales); }
    }
    else if (tiles_per_cu >= 2)
    {
        if (a.tokens <= 8) { launch_gemv4_mfma<BLOCK, 1, 1, 8>(t, scales); }
        else { launch_gemv4_mfma<BLOCK, 4, 1, 8>(t, scales); }
    }
    else if (a.K > 8192 && a.tokens <= 4) { launch_gemv4_mfma<BLOCK, 1, 2, 16>(t, scales); }
    else { launch_gemv4_mfma<BLOCK, 1, 1, 16>(t, scales); }
    return true;
}

// Where the matrix-core kernel beats the dot2 kernel on the same weight: from three tokens on (one pass instead of a
// pass per four tokens; 4096 x 14336 at four tokens 9.1 us against 13.2), and for long rows with few row tiles even
// at one token (14336 x 4096: 8.4 us against 9.0).
inline bool fp4_tiled_pays(const LinearArgs& a)
{
    return a.tokens >= 3 || (a.K > 8192 && ((a.n_out + 15) / 16) / cu_count() < 2);
}

template <int MT, int R, int U, int WAVES, int OCC, int BLOCK>
bool launch_gemv4_dot2(const LinearArgs& a)
{
    const size_t lds = (size_t)MT * ((a.K + 2047) / 2048) * 4096;
    auto kernel = gemv4_dot2_kernel<MT, R, U, WAVES, BLOCK>;
    if (!allow_big_lds(kernel, lds)) { return false; }
    const int want = ((a.n_out + R - 1) / R + WAVES - 1) / WAVES;
    const int cap = cu_count() * (lds > 80 * 1024 ? 1 : (lds > 40 * 1024 && OCC > 2 ? 2 : OCC));
    kernel<<<want < cap ? want : cap, WAVES * 64, lds, stream()>>>(a);
    return true;
}

// Tuned on MI355X (block 16, one token) with rotating weight buffers.
template <int MT, int BLOCK>
bool pick_gemv4_dot2(const LinearArgs& a)
{
    const long long bytes = (long long)a.n_out * a.K / 2;
    if (bytes <= (8LL << 20)) { return launch_gemv4_dot2<MT, 1, 4, 8, 2, BLOCK>(a); }
    if (a.K > 8192) { return launch_gemv4_dot2<MT, 2, 4, 8, 2, BLOCK>(a); }
    if (a.n_out / cu_count() >= 128) { return launch_gemv4_dot2<MT, 2, 2, 4, 4, BLOCK>(a); }
    return launch_gemv4_dot2<MT, 2, 4, 4, 4, BLOCK>(a);
}

// Rows of K % 32 == 16 elements (blocks of 16): the ragged instantiation, one shape for every size
template <int MT>
bool launch_gemv4_dot2_ragged(const LinearArgs& a)
{
    const size_t lds = (size_t)MT * ((a.K + 2047) / 2048) * 4096;
    auto kernel = gemv4_dot2_kernel<MT, 1, 2, 8, 16, true>;
    if (!allow_big_lds(kernel, lds)) { return false; }
    const int want = (a.n_out + 7) / 8;
    const int cap = cu_count() * (lds > 80 * 1024 ? 1 : 2);
    kernel<<<want < cap ? want : cap, 512, lds, stream()>>>(a);
    return true;
}

bool gemv4_dot2_ragged(const LinearArgs& a)
{
    switch (a.tokens)
    {
    case 1: return launch_gemv4_dot2_ragged<1>(a);
    case 2: return launch_gemv4_dot2_ragged<2>(a);
    case 3: return launch_gemv4_dot2_ragged<3>(a);
    case 4: return launch_gemv4_dot2_ragged<4>(a);
    default: return false;
    }
}

template <int BLOCK>
bool gemv4_dot2(const LinearArgs& a)
{
    switch (a.tokens)
    {
    case 1: return pick_gemv4_dot2<1, BLOCK>(a);
    case 2: return pick_gemv4_dot2<2, BLOCK>(a);
    case 3: return pick_gemv4_dot2<3, BLOCK>(a);
    case 4: return pick_gemv4_dot2<4, BLOCK>(a);
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

const unsigned char* ccq::lookup_tiled(const void* W, int type, int n_out, int K, long long ldw)
{
    std::shared_lock<std::shared_mutex> lock(g_tiled_mutex);
    if (g_tiled.empty()) { return nullptr; }
    const auto it = g_tiled.find(W);
    if (it == g_tiled.end()) { return nullptr; }
    const TiledWeight& t = it->second;
    return (t.type == type && t.n_out == n_out && t.K == K && t.ldw == ldw) ? t.tiled : nullptr;
}

namespace
{

// Device address of `scratch` on the current device (the array's name is only a host-side handle), looked up
// once per device with that device current.
float* static_scratch()
{
    constexpr int kMaxDevices = 64;
    static std::mutex mutex;
    static void* ptr[kMaxDevices] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
    {
        (void)hipGetLastError();
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(mutex);
    if (!ptr[dev])
    {
        void* p = nullptr;
        const hipError_t err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (err != hipSuccess || !p)
        {
            fprintf(stderr, "hip_quant_gemm_noalloc: hipGetSymbolAddress failed on device %d: %s\n", dev, hipGetErrorString(err));
            (void)hipGetLastError();
            return nullptr;
        }
        ptr[dev] = p;
    }
    return (float*)ptr[dev];
}

int quant_gemm(int transA, int transB, int M, int N, int K, float alpha,
               const void* A, int typeA, int lda, float invScaleA,
               const void* B, int typeB, int ldb, float invScaleB,
               float beta, void* C, int typeC, int ldc,
               const void* blk_scA, const void* blk_scB, unsigned int block_size, SplitScratch* split_scratch)
{
    const bool aQ = is_quantized(typeA), bQ = is_quantized(typeB);
    if (aQ == bQ) { return -1; }
    // the unquantized operand and C share one 16-bit type: BF16 (cccc/cublas_real.h:943-964) or HALF (:921-938, FP8 weights only)
    const int act_type = aQ ? typeB : typeA;
    if ((act_type != DT_BF16 && act_type != DT_HALF) || typeC != act_type) { return -1; }
    if (act_type == DT_HALF && (aQ ? typeA : typeB) == DT_FP4) { return -1; }
    if ((transA != 0 && transA != 1) || (transB != 0 && transB != 1)) { return -1; }
    if (M < 0 || N < 0 || K < 0 || lda <= 0 || ldb <= 0 || ldc <= 0) { return -1; }
    if (M == 0 || N == 0) { return 0; }
    if (!A || !B || !C) { return -1; }

    GenericArgs g{};
    g.act_type = act_type;
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
        if (act_type == DT_HALF)
        {
            if (x_ok && K % 16 == 0 && a.ldw % 16 == 0 && aligned16(a.W))
            {
                const char* name = half_linear(a, g.w_type, split_scratch);
                if (!name) { return -2; }
                note_kernel(name);
                launched = true;
            }
        }
        else if (g.w_type == DT_FP4)
        {
            const bool ok = x_ok && a.blk_sc && (a.block_size == 16 || a.block_size == 32) && K % 32 == 0 && a.ldw % 32 == 0 &&
                            aligned16(a.W) && ((uintptr_t)a.blk_sc & 1u) == 0;
            // blocks of 16 over the flat index with K % 32 == 16 (dense rows): the ragged dot2 kernel, up to 16 tokens
            const bool ragged = !ok && x_ok && a.blk_sc && a.block_size == 16 && K % 32 == 16 && a.ldw == K && aligned16(a.W) && a.tokens <= 16;
            if (ragged)
            {
                launched = true;
                for (int t0 = 0; t0 < g.tokens && launched; t0 += 4)
                {
                    LinearArgs s = a;
                    s.tokens = (g.tokens - t0 < 4) ? g.tokens - t0 : 4;
                    s.X = a.X + (long long)t0 * a.ldx;
                    s.Y = a.Y + (long long)t0 * a.y_stride_tok;
                    launched = gemv4_dot2_ragged(s);
                }
                if (launched) { note_kernel("gemv_dot2"); }
            }
            if (ok && a.tokens <= 16)
            {
                const uint8_t* tiled = fp4_tiled_pays(a) ? find_tiled_fp4(a) : nullptr;
                if (tiled)
                {
                    launched = a.block_size == 16 ? gemv4_mfma_tiled<16>(a, tiled) : gemv4_mfma_tiled<32>(a, tiled);
                    if (launched) { note_kernel("gemv_mfma_tiled"); }
                }
            }
            if (ok && a.tokens <= 16 && !launched)
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
            else if (ok && !launched)
            {
                // the register-fed kernel reads the tiled copy; it wants whole 128-element chunks
                const uint8_t* tiled = (K % 128 == 0 && a.tokens >= 17) ? find_tiled_fp4(a) : nullptr;
                launched = a.block_size == 16 ? gemm_mfma<DT_FP4, 16>(a, tiled, split_scratch) : gemm_mfma<DT_FP4, 32>(a, tiled, split_scratch);
                if (!launched) { return -2; }                    // only a fixed scratch buffer that is too small ends here
                note_kernel(tiled ? "gemm_mfma_tiled" : "gemm_mfma");
            }
        }
        else
        {
            const bool ok = x_ok && K % 16 == 0 && a.ldw % 16 == 0 && aligned16(a.W);
            const bool scaled = a.w_scale != 1.0f;
            // With a tiled copy registered for this weight the matrix-core kernel on that copy is the fastest
            // choice for every token count up to 16 (3-17 % faster than the dot2 kernels at one and two tokens,
            // more above), except one or two tokens on weights of a few MiB, where the software-pipelined dot2
            // kernel starts sooner.
            if (ok && a.tokens <= 16 && (a.tokens >= 3 || (long long)a.n_out * K >= (8LL << 20)))
            {
                if (const uint8_t* tiled = find_tiled(a, g.w_type))
                {
                    if (g.w_type == DT_E5M2) { launched = scaled ? gemv8_mfma_ksplit_tiled<DT_E5M2, true>(a, tiled) : gemv8_mfma_ksplit_tiled<DT_E5M2, false>(a, tiled); }
                    else { launched = scaled ? gemv8_mfma_ksplit_tiled<DT_E4M3, true>(a, tiled) : gemv8_mfma_ksplit_tiled<DT_E4M3, false>(a, tiled); }
                    if (launched) { note_kernel("gemv_mfma_tiled"); }
                }
            }
            if (ok && !launched && a.tokens <= 4)
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
                const uint8_t* tiled = find_tiled(a, g.w_type);
                if (g.w_type == DT_E5M2) { launched = gemm_mfma<DT_E5M2, 0>(a, tiled, split_scratch); }
                else { launched = gemm_mfma<DT_E4M3, 0>(a, tiled, split_scratch); }
                if (!launched) { return -2; }                    // only a fixed scratch buffer that is too small ends here
                note_kernel(tiled ? "gemm_mfma_tiled" : "gemm_mfma");
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

}    // namespace

int hip_quant_gemm(int transA, int transB, int M, int N, int K, float alpha,
                   const void* A, int typeA, int lda, float invScaleA,
                   const void* B, int typeB, int ldb, float invScaleB,
                   float beta, void* C, int typeC, int ldc, float /*act_scale*/,
                   const void* blk_scA, const void* blk_scB, unsigned int block_size)
{
    return quant_gemm(transA, transB, M, N, K, alpha, A, typeA, lda, invScaleA, B, typeB, ldb, invScaleB, beta, C, typeC, ldc,
                      blk_scA, blk_scB, block_size, nullptr);
}

int hip_quant_gemm_segments(int n_segments, const int* n_out, const void* const* W, const float* inv_scale, void* const* Y, const int* ldy,
                            int w_type, int tokens, int K, int ldw, const void* X, int ldx)
{
    const bool fp4 = w_type == DT_FP4;
    if (w_type != DT_E5M2 && w_type != DT_E4M3 && !fp4) { return -1; }
    if (fp4 && (K % 128 != 0 || ldw != K)) { return -1; }
    if (n_segments < 1 || n_segments > 3 || !n_out || !W || !inv_scale || !Y || !ldy) { return -1; }
    if (tokens < 2 || K <= 0 || K % 64 != 0 || ldw < K || ldx < K || !X || !aligned16(X) || ldw % 16 != 0 || ldx % 8 != 0) { return -1; }
    if ((long long)tokens * ldx * 2 >= (1LL << 32)) { return -1; }
    LinearArgs a{};
    a.X = (const uint16_t*)X;
    a.ldw = ldw;
    a.ldx = ldx;
    a.y_stride_out = 1;
    a.tokens = tokens;
    a.K = K;
    a.alpha = 1.0f;
    a.beta = 0.0f;
    a.n_segments = n_segments;
    bool all_tiled = true;
    const uint8_t* tiled[3] = { nullptr, nullptr, nullptr };
    for (int s = 0; s < n_segments; s++)
    {
        if (n_out[s] <= 0 || !W[s] || !Y[s] || !aligned16(W[s]) || ldy[s] < n_out[s] || (long long)n_out[s] * ldw >= (1LL << 32)) { return -1; }
        a.seg_W[s] = (const uint8_t*)W[s];
        a.seg_Y[s] = (uint16_t*)Y[s];
        a.seg_n_out[s] = n_out[s];
        a.seg_w_scale[s] = inv_scale[s];
        a.seg_y_stride_tok[s] = ldy[s];
        tiled[s] = ccq::lookup_tiled(W[s], w_type, n_out[s], K, ldw);
        all_tiled = all_tiled && tiled[s] != nullptr;
    }
    if (fp4)
    {
        // FP4 runs on the tiled copies only (codes, then the scale bytes): the block length comes from the registration
        if (!all_tiled) { return -1; }
        const unsigned block = tiled_block_of(W[0]);
        for (int s = 0; s < n_segments; s++)
        {
            if (tiled_block_of(W[s]) != block) { return -1; }
            a.seg_W[s] = tiled[s];
        }
        note_kernel("gemm_segments_tiled");
        if (block == 16) { launch_gemm4_mfma_direct_segments<16>(a); }
        else if (block == 32) { launch_gemm4_mfma_direct_segments<32>(a); }
        else { return -1; }
        return finish("quant_gemm_segments");
    }
    // every weight on its tiled copy, or every weight on the file layout
    if (all_tiled)
    {
        for (int s = 0; s < n_segments; s++) { a.seg_W[s] = tiled[s]; }
        note_kernel("gemm_segments_tiled");
        if (w_type == DT_E5M2) { launch_gemm_mfma_direct_segments<DT_E5M2, true>(a); }
        else { launch_gemm_mfma_direct_segments<DT_E4M3, true>(a); }
    }
    else
    {
        note_kernel("gemm_segments");
        if (w_type == DT_E5M2) { launch_gemm_mfma_direct_segments<DT_E5M2, false>(a); }
        else { launch_gemm_mfma_direct_segments<DT_E4M3, false>(a); }
    }
    return finish("quant_gemm_segments");
}

int hip_quant_gemm_swiglu(int n_out, int tokens, int K, const void* W_gate, const void* W_up, int w_type, int ldw,
                          float inv_scale_gate, float inv_scale_up, const void* X, int ldx, void* Y, int ldy)
{
    const bool fp4 = w_type == DT_FP4;
    if (w_type != DT_E5M2 && w_type != DT_E4M3 && !fp4) { return -1; }
    if (fp4 && (K % 128 != 0 || ldw != K)) { return -1; }
    if (n_out <= 0 || tokens < 2 || K <= 0 || K % 64 != 0 || ldw < K || ldx < K || ldy < n_out) { return -1; }
    if (!W_gate || !W_up || !X || !Y || !aligned16(W_gate) || !aligned16(W_up) || !aligned16(X) || ldw % 16 != 0 || ldx % 8 != 0) { return -1; }
    if ((long long)n_out * ldw >= (1LL << 32) || (long long)tokens * ldx * 2 >= (1LL << 32)) { return -1; }
    LinearArgs a{};
    a.W = (const uint8_t*)W_gate;
    a.W_pair = (const uint8_t*)W_up;
    a.X = (const uint16_t*)X;
    a.Y = (uint16_t*)Y;
    a.ldw = ldw;
    a.ldx = ldx;
    a.y_stride_tok = ldy;
    a.y_stride_out = 1;
    a.n_out = n_out;
    a.tokens = tokens;
    a.K = K;
    a.w_scale = inv_scale_gate;
    a.w_scale_pair = inv_scale_up;
    a.alpha = 1.0f;
    a.beta = 0.0f;
    // both weights on their tiled copies, or both on the file layout
    const uint8_t* tg = ccq::lookup_tiled(W_gate, w_type, n_out, K, ldw);
    const uint8_t* tu = tg ? ccq::lookup_tiled(W_up, w_type, n_out, K, ldw) : nullptr;
    if (fp4)
    {
        // FP4 runs on the tiled copies only (codes, then the scale bytes), both of one block length
        if (!tg || !tu) { return -1; }
        const unsigned block = tiled_block_of(W_gate);
        if (tiled_block_of(W_up) != block) { return -1; }
        a.W = tg;
        a.W_pair = tu;
        note_kernel("gemm_swiglu_tiled");
        if (block == 16) { launch_gemm4_mfma_direct_pair<16>(a); }
        else if (block == 32) { launch_gemm4_mfma_direct_pair<32>(a); }
        else { return -1; }
        return finish("quant_gemm_swiglu");
    }
    if (tg && tu)
    {
        a.W = tg;
        a.W_pair = tu;
        note_kernel("gemm_swiglu_tiled");
        if (w_type == DT_E5M2) { launch_gemm_mfma_direct_pair<DT_E5M2, true>(a); }
        else { launch_gemm_mfma_direct_pair<DT_E4M3, true>(a); }
    }
    else
    {
        note_kernel("gemm_swiglu");
        if (w_type == DT_E5M2) { launch_gemm_mfma_direct_pair<DT_E5M2, false>(a); }
        else { launch_gemm_mfma_direct_pair<DT_E4M3, false>(a); }
    }
    return finish("quant_gemm_swiglu");
}

int hip_quant_gemm_add_rms_norm(int n_out, int tokens, int K, const void* W, int w_type, int ldw, float inv_scale, const void* X, int ldx,
                                const void* res, void* sum, const void* norm_w, void* y, float epsilon)
{
    const bool fp4 = w_type == DT_FP4;
    if (w_type != DT_E5M2 && w_type != DT_E4M3 && !fp4) { return -1; }
    if (fp4 && (K % 128 != 0 || ldw != K)) { return -1; }
    if (n_out <= 0 || n_out % 8 != 0 || n_out > 4096 || tokens < 2 || K <= 0 || K % 64 != 0 || ldw < K || ldx < K) { return -1; }
    if (!W || !X || !res || !sum || !norm_w || !y || ldw % 16 != 0 || ldx % 8 != 0) { return -1; }
    if (!aligned16(W) || !aligned16(X) || !aligned16(res) || !aligned16(sum) || !aligned16(norm_w) || !aligned16(y)) { return -1; }
    LinearArgs a{};
    a.W = (const uint8_t*)W;
    a.X = (const uint16_t*)X;
    a.ldw = ldw;
    a.ldx = ldx;
    a.y_stride_tok = n_out;
    a.y_stride_out = 1;
    a.n_out = n_out;
    a.tokens = tokens;
    a.K = K;
    a.w_scale = inv_scale;
    a.alpha = 1.0f;
    a.beta = 0.0f;
    const AddNormArgs e = { (const uint16_t*)res, (uint16_t*)sum, (const uint16_t*)norm_w, (uint16_t*)y, epsilon };
    const uint8_t* tiled = ccq::lookup_tiled(W, w_type, n_out, K, ldw);
    bool launched = false;
    if (fp4)
    {
        if (!tiled) { return -1; }
        const unsigned block = tiled_block_of(W);
        a.block_size = block;
        if (block == 16) { launched = gemm_mfma<DT_FP4, 16>(a, tiled, nullptr, &e); }
        else if (block == 32) { launched = gemm_mfma<DT_FP4, 32>(a, tiled, nullptr, &e); }
    }
    else if (w_type == DT_E5M2) { launched = gemm_mfma<DT_E5M2, 0>(a, tiled, nullptr, &e); }
    else { launched = gemm_mfma<DT_E4M3, 0>(a, tiled, nullptr, &e); }
    if (!launched) { return -1; }                   // this shape does not split its k range: nothing to fold the add and the norm into
    note_kernel(tiled ? "gemm_add_rms_norm_tiled" : "gemm_add_rms_norm");
    return finish("quant_gemm_add_rms_norm");
}

int hip_quant_gemm_noalloc(int transA, int transB, int M, int N, int K, float alpha,
                           const void* A, int typeA, int lda, float invScaleA,
                           const void* B, int typeB, int ldb, float invScaleB,
                           float beta, void* C, int typeC, int ldc, float /*act_scale*/,
                           const void* blk_scA, const void* blk_scB, unsigned int block_size)
{
    SplitScratch fixed;
    fixed.strict = true;
    fixed.fixed = static_scratch();
    fixed.fixed_bytes = HIP_QUANT_NOALLOC_SCRATCH_BYTES;
    const int rc = quant_gemm(transA, transB, M, N, K, alpha, A, typeA, lda, invScaleA, B, typeB, ldb, invScaleB, beta, C, typeC, ldc,
                              blk_scA, blk_scB, block_size, &fixed);
    if (rc == -2 && !fixed.fixed) { return 1; }      // the symbol lookup failed and said so
    if (rc == -2)
    {
        fprintf(stderr, "hip_quant_gemm_noalloc: this shape splits K over workgroups and needs %zu bytes of partial sums; "
                        "the static scratch holds %llu (nothing was launched)\n",
                fixed.refused, (unsigned long long)HIP_QUANT_NOALLOC_SCRATCH_BYTES);
        return -1;
    }
    return rc;
}

unsigned long long hip_quant_tiled_size(int type, int n_out, int K)
{
    if (n_out <= 0 || K <= 0) { return 0ull; }
    const unsigned long long tiles = (unsigned long long)((n_out + 15) / 16);
    // FP4: a KiB of codes and up to 128 scale bytes per 16 rows x 128 elements
    if (type == DT_FP4) { return tiles * (unsigned long long)((K + 127) / 128) * (1024ull + 128ull); }
    if (type != DT_E4M3 && type != DT_E5M2) { return 0ull; }
    return tiles * (unsigned long long)((K + 63) / 64) * 1024ull;
}

int hip_quant_weight_prepare_fp4(const void* W, const void* blk_sc, unsigned int block_size, int n_out, int K, void* dst_tiled)
{
    if (!W || !blk_sc || !dst_tiled || n_out <= 0 || K <= 0 || (block_size != 16 && block_size != 32)) { return -1; }
    if (K % 32 != 0 || !aligned16(W) || !aligned16(dst_tiled)) { return -1; }
    const long long n_units = (long long)((n_out + 15) / 16) * ((K + 127) / 128) * 64;
    long long blocks = (n_units + 255) / 256;
    const long long cap = (long long)cu_count() * 16;
    if (blocks > cap) { blocks = cap; }
    repack_tiled_fp4_kernel<<<(unsigned)blocks, 256, 0, stream()>>>((const uint8_t*)W, (const uint8_t*)blk_sc, (uint8_t*)dst_tiled, n_out, K, (int)block_size);
    const int rc = finish("weight_prepare_fp4");
    if (rc != 0) { return rc; }
    std::unique_lock<std::shared_mutex> lock(g_tiled_mutex);
    g_tiled[W] = TiledWeight{ (const uint8_t*)dst_tiled, DT_FP4, n_out, K, (long long)K, blk_sc, block_size };
    return 0;
}

int hip_quant_weight_prepare(const void* W, int type, int n_out, int K, int ldw, void* dst_tiled)
{
    if ((type != DT_E4M3 && type != DT_E5M2) || !W || !dst_tiled || n_out <= 0 || K <= 0) { return -1; }
    if (K % 16 != 0 || ldw % 16 != 0 || ldw < K || !aligned16(W) || !aligned16(dst_tiled)) { return -1; }
    const long long n_chunks = (long long)((n_out + 15) / 16) * ((K + 63) / 64) * 64;
    long long blocks = (n_chunks + 255) / 256;
    const long long cap = (long long)cu_count() * 16;
    if (blocks > cap) { blocks = cap; }
    repack_tiled_kernel<<<(unsigned)blocks, 256, 0, stream()>>>((const uint8_t*)W, (uint8_t*)dst_tiled, n_out, K, ldw);
    const int rc = finish("weight_prepare");
    if (rc != 0) { return rc; }
    std::unique_lock<std::shared_mutex> lock(g_tiled_mutex);
    g_tiled[W] = TiledWeight{ (const uint8_t*)dst_tiled, type, n_out, K, (long long)ldw, nullptr, 0u };
    return 0;
}

int hip_quant_weight_release(const void* W)
{
    std::unique_lock<std::shared_mutex> lock(g_tiled_mutex);
    g_tiled.erase(W);
    return 0;
}
