// C-ABI entry points of the decode-step neighbours (kernels in decode_kernels.h).
#include "../../include/cccc_hip_quant.h"
#include "decode_kernels.h"
#include "runtime.h"
#include <cstdio>

using namespace ccq;

namespace
{

inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

template <int WT, bool SCALED>
int launch_fused(const FusedLinearArgs& a, int n_groups)
{
    const size_t lds = (size_t)((a.K + 1023) / 1024) * 2048;
    if (lds > 64 * 1024) { return -1; }
    const int cus = cu_count();
    // Configurations chosen by whole-step time of the Qwen3-8B decode, which resolves 0.05 us per launch (the kernels
    // timed alone prefer other settings, e.g. 8 waves for long rows).
    const int want4 = (n_groups + 3) / 4;
    if (!a.norm_w && a.K % 1024 == 0 && n_groups < cus * 64)
    {
        // nothing to normalise: x comes with the weights, no LDS.  Long rows in batches of 2 KiB per row, rows of up to
        // 4 KiB in one request.
        if (a.K > 4096) { gemv8_fused_kernel<WT, 2, 4, SCALED, true><<<want4 < cus * 4 ? want4 : cus * 4, 256, 0, stream()>>>(a); }
        else { gemv8_fused_kernel<WT, 4, 4, SCALED, true><<<want4 < cus * 2 ? want4 : cus * 2, 256, 0, stream()>>>(a); }
    }
    else if (a.K > 8192 && n_groups < cus * 64)
    {
        gemv8_fused_kernel<WT, 4, 4, SCALED><<<want4 < cus * 2 ? want4 : cus * 2, 256, lds, stream()>>>(a);
    }
    // very tall weights want 8-wave workgroups, as the plain GEMV dispatch found
    else if (n_groups >= cus * 64)
    {
        const int want = (n_groups + 7) / 8;
        gemv8_fused_kernel<WT, 4, 8, SCALED><<<want < cus * 2 ? want : cus * 2, 512, lds, stream()>>>(a);
    }
    else if (a.K <= 4096)
    {
        // short rows: two batches of 2 KiB per row pair keep the next request ahead of the multiply (measured 5-10 % faster than one batch of 4)
        gemv8_fused_kernel<WT, 2, 4, SCALED><<<want4 < cus * 4 ? want4 : cus * 4, 256, lds, stream()>>>(a);
    }
    else
    {
        gemv8_fused_kernel<WT, 4, 4, SCALED><<<want4 < cus * 4 ? want4 : cus * 4, 256, lds, stream()>>>(a);
    }
    return finish("quant_linear_fused");
}

// BF16 weights (a tied lm_head): the dot2 kernel on 2-byte elements; launch shapes as for FP8 rows of twice the length.
int launch_fused_bf16(const FusedLinearArgs& a, int n_groups)
{
    const size_t lds = (size_t)((a.K + 511) / 512) * 1024;
    if (lds > 64 * 1024) { return -1; }
    const int cus = cu_count();
    if (n_groups >= cus * 64)
    {
        const int want = (n_groups + 7) / 8;
        gemv8_fused_kernel<DT_BF16, 4, 8, false><<<want < cus * 2 ? want : cus * 2, 512, lds, stream()>>>(a);
    }
    else
    {
        const int want4 = (n_groups + 3) / 4;
        gemv8_fused_kernel<DT_BF16, 4, 4, false><<<want4 < cus * 4 ? want4 : cus * 4, 256, lds, stream()>>>(a);
    }
    return finish("quant_linear_fused");
}

// FP4 block-scale weights: two rows per wave, U = 2 batches for rows of up to 4096 elements (one k-step of 2048 per
// lane and row is 1 KiB), 8-wave workgroups for very tall weights, as for FP8.
template <int BLOCK>
int launch_fused_fp4(const FusedLinearArgs& a, int n_groups)
{
    const size_t lds = (size_t)((a.K + 2047) / 2048) * 4096;
    if (lds > 64 * 1024) { return -1; }
    const int cus = cu_count();
    const int want4 = (n_groups + 3) / 4;
    if (n_groups >= cus * 64)
    {
        const int want = (n_groups + 7) / 8;
        gemv4_fused_kernel<BLOCK, 2, 8><<<want < cus * 2 ? want : cus * 2, 512, lds, stream()>>>(a);
    }
    else if (a.K <= 8192) { gemv4_fused_kernel<BLOCK, 1, 4><<<want4 < cus * 4 ? want4 : cus * 4, 256, lds, stream()>>>(a); }
    else { gemv4_fused_kernel<BLOCK, 2, 4><<<want4 < cus * 4 ? want4 : cus * 4, 256, lds, stream()>>>(a); }
    return finish("quant_linear_fused");
}

// Matrix-core variant on the tiled copies.  Configurations from the tuning of gemv8_mfma_kernel at one token.
template <int WT, int RT, int U, int WAVES, bool SCALED>
void launch_fused_mfma_cfg(const FusedLinearArgs& a, int n_tiles, size_t lds)
{
    if (a.norm_w) { gemv8_fused_mfma_kernel<WT, RT, U, WAVES, SCALED, true><<<(n_tiles + RT - 1) / RT, WAVES * 64, lds, stream()>>>(a); }
    else { gemv8_fused_mfma_kernel<WT, RT, U, WAVES, SCALED, false><<<(n_tiles + RT - 1) / RT, WAVES * 64, 0, stream()>>>(a); }
}

template <int WT, bool SCALED>
int launch_fused_mfma(const FusedLinearArgs& a, int n_tiles)
{
    const size_t lds = (size_t)((a.K + 1023) / 1024) * 2048;
    if (lds > 48 * 1024) { return -1; }
    const int tiles_per_cu = n_tiles / cu_count();
    if (tiles_per_cu >= 16) { launch_fused_mfma_cfg<WT, 2, 2, 8, SCALED>(a, n_tiles, lds); }
    else if (tiles_per_cu >= 2) { launch_fused_mfma_cfg<WT, 1, 1, 8, SCALED>(a, n_tiles, lds); }
    else if (a.K > 8192) { launch_fused_mfma_cfg<WT, 1, 4, 8, SCALED>(a, n_tiles, lds); }
    else { launch_fused_mfma_cfg<WT, 1, 2, 16, SCALED>(a, n_tiles, lds); }
    return finish("quant_linear_fused");
}

}    // namespace

int hip_quant_linear_fused(const hip_fused_linear* d)
{
    if (!d || (d->w_type != DT_E4M3 && d->w_type != DT_E5M2 && d->w_type != DT_FP4 && d->w_type != DT_BF16)) { return -1; }
    if (d->K <= 0 || d->K % 16 != 0 || d->n_segments < 1 || d->n_segments > 3 || !d->X || !aligned16(d->X)) { return -1; }
    const bool fp4 = d->w_type == DT_FP4;
    if (fp4 && (d->K % 32 != 0 || (d->block_size != 16 && d->block_size != 32))) { return -1; }
    if (d->pair && d->n_segments != 2) { return -1; }
    if (d->residual && !d->pair && d->n_segments != 1) { return -1; }
    if (d->norm_weight && !aligned16(d->norm_weight)) { return -1; }
    FusedLinearArgs a{};
    bool scaled = false;
    int n_groups = 0;
    for (int s = 0; s < d->n_segments; s++)
    {
        if (!d->W[s] || !aligned16(d->W[s]) || d->n_out[s] <= 0) { return -1; }
        if (!d->pair && !d->Y[s]) { return -1; }
        if (fp4 && (!d->blk_sc[s] || ((uintptr_t)d->blk_sc[s] & 1u))) { return -1; }
        a.W[s] = (const uint8_t*)d->W[s];
        a.S[s] = fp4 ? (const uint8_t*)d->blk_sc[s] : nullptr;
        a.Y[s] = (uint16_t*)d->Y[s];
        a.n_out[s] = d->n_out[s];
        a.w_scale[s] = d->w_scale[s];
        scaled = scaled || d->w_scale[s] != 1.0f;
        n_groups += (d->n_out[s] + 1) / 2;
    }
    if (d->pair)
    {
        if (d->n_out[1] != d->n_out[0] || !d->Y[0]) { return -1; }
        n_groups = d->n_out[0];
    }
    a.n_segments = d->n_segments;
    a.pair = d->pair ? 1 : 0;
    a.K = d->K;
    a.X = (const uint16_t*)d->X;
    a.norm_w = (const uint16_t*)d->norm_weight;
    a.norm_eps = d->norm_eps;
    a.residual = (const uint16_t*)d->residual;
    a.block = d->block_size;
    if (d->argmax_workspace && (d->n_segments != 1 || d->pair || !aligned16(d->argmax_workspace))) { return -1; }
    a.argmax_ws = d->argmax_workspace;
    if (d->w_type == DT_BF16)
    {
        if (scaled) { return -1; }                          // a plain BF16 weight carries no dequantisation scale
        note_kernel("gemv_fused_bf16");
        return launch_fused_bf16(a, n_groups);
    }
    if (fp4)
    {
        note_kernel("gemv_fused_fp4");
        return d->block_size == 16 ? launch_fused_fp4<16>(a, n_groups) : launch_fused_fp4<32>(a, n_groups);
    }
    // every segment has a registered tiled copy (and this is not the SwiGLU pair): matrix-core variant
    if (!d->pair)
    {
        int n_tiles = 0;
        bool all = true;
        for (int s = 0; s < d->n_segments && all; s++)
        {
            a.T[s] = lookup_tiled(d->W[s], d->w_type, d->n_out[s], d->K, d->K);
            all = a.T[s] != nullptr;
            n_tiles += (d->n_out[s] + 15) / 16;
        }
        // measured inside the decode step: on tall weights the matrix-core variant wins (lm_head 91 us against 97);
        // on the per-layer weights it is level with the dot2 kernel without a norm in front (o 5.6 against 5.9 us,
        // down 11.4 against 11.45) and slower with one (q,k,v 10.5 against 7.3), so those stay on the row-major bytes
        if (all && n_tiles / cu_count() < 16) { all = false; }
        if (all)
        {
            note_kernel("gemv_fused_mfma");
            int rc;
            if (d->w_type == DT_E5M2) { rc = scaled ? launch_fused_mfma<DT_E5M2, true>(a, n_tiles) : launch_fused_mfma<DT_E5M2, false>(a, n_tiles); }
            else { rc = scaled ? launch_fused_mfma<DT_E4M3, true>(a, n_tiles) : launch_fused_mfma<DT_E4M3, false>(a, n_tiles); }
            if (rc >= 0) { return rc; }
        }
    }
    note_kernel("gemv_fused");
    if (d->w_type == DT_E5M2) { return scaled ? launch_fused<DT_E5M2, true>(a, n_groups) : launch_fused<DT_E5M2, false>(a, n_groups); }
    return scaled ? launch_fused<DT_E4M3, true>(a, n_groups) : launch_fused<DT_E4M3, false>(a, n_groups);
}

int hip_rms_norm_fwd(int type, void* X, void* Y, void* scale, void* invstd_out, unsigned int outer, unsigned int inner, float epsilon)
{
    if (type != DT_BF16)
    {
        fprintf(stderr, "hip_rms_norm_fwd: unsupported type=%d\n", type);
        return 1;
    }
    if (outer == 0 || inner == 0) { return 0; }
    if (!X || !Y || !scale)
    {
        fprintf(stderr, "hip_rms_norm_fwd: null pointer\n");
        return 1;
    }
    const uint16_t *x = (const uint16_t*)X, *w = (const uint16_t*)scale;
    uint16_t* y = (uint16_t*)Y;
    if (inner > 64u * 8u * RMS_CHUNKS) { rms_norm_long_rows_kernel<<<outer, 256, 0, stream()>>>(x, y, w, (float*)invstd_out, inner, epsilon); }
    else if (inner % 8 == 0 && aligned16(X) && aligned16(Y) && aligned16(scale)) { rms_norm_rows_kernel<true><<<(outer + 3) / 4, 256, 0, stream()>>>(x, y, w, (float*)invstd_out, outer, inner, epsilon); }
    else { rms_norm_rows_kernel<false><<<(outer + 3) / 4, 256, 0, stream()>>>(x, y, w, (float*)invstd_out, outer, inner, epsilon); }
    return finish("rms_norm_fwd_bf16");
}

int hip_rope_fwd(int type, const void* X, void* Y, const void* cos_tab, const void* sin_tab, unsigned int D, unsigned int T, unsigned int B, unsigned int pos_offset)
{
    if (D % 2 != 0)
    {
        fprintf(stderr, "hip_rope_fwd: D must be even (D=%u)\n", D);
        return 1;
    }
    if (type != DT_BF16)
    {
        fprintf(stderr, "hip_rope_fwd: unsupported type=%d\n", type);
        return 1;
    }
    const unsigned total = (D / 2) * T * B;
    if (total == 0) { return 0; }
    if (!X || !Y || !cos_tab || !sin_tab)
    {
        fprintf(stderr, "hip_rope_fwd: null pointer\n");
        return 1;
    }
    const bool vec = (D / 2) % 8 == 0 && aligned16(X) && aligned16(Y) && aligned16(cos_tab) && aligned16(sin_tab);
    const unsigned items = vec ? total / 8 : total;
    if (vec) { rope_rows_kernel<true><<<(items + 255) / 256, 256, 0, stream()>>>((const uint16_t*)X, (uint16_t*)Y, (const uint16_t*)cos_tab, (const uint16_t*)sin_tab, D, T, T * B, pos_offset); }
    else { rope_rows_kernel<false><<<(items + 255) / 256, 256, 0, stream()>>>((const uint16_t*)X, (uint16_t*)Y, (const uint16_t*)cos_tab, (const uint16_t*)sin_tab, D, T, T * B, pos_offset); }
    return finish("rope_fwd_bf16");
}

int hip_embed_fwd(int type, const void* ids, const void* W, void* Y, int D, int T, int B)
{
    if (type != DT_BF16 || D <= 0 || D % 8 != 0)
    {
        fprintf(stderr, "hip_embed_fwd: unsupported type=%d or D=%d\n", type, D);
        return 1;
    }
    if (T * B <= 0) { return 0; }
    if (!ids || !W || !Y)
    {
        fprintf(stderr, "hip_embed_fwd: null pointer\n");
        return 1;
    }
    embed_bf16_kernel<<<dim3(1, T * B), 256, 0, stream()>>>((const float*)ids, nullptr, (const uint16_t*)W, (uint16_t*)Y, D, 0x7FFFFFFF);
    return finish("embed_fwd_bf16");
}

int hip_embed_token_bf16(const void* d_token, const void* W, void* y, int D, int n_rows)
{
    if (!d_token || !W || !y || D <= 0 || D % 8 != 0 || n_rows <= 0) { return -1; }
    embed_bf16_kernel<<<dim3(1, 1), 256, 0, stream()>>>(nullptr, (const int*)d_token, (const uint16_t*)W, (uint16_t*)y, D, n_rows);
    return finish("embed_token_bf16");
}

int hip_qk_norm_rope_kv_bf16(const void* q, const void* k, const void* v, const void* q_norm_w, const void* k_norm_w,
                             const void* cos_tab, const void* sin_tab, void* q_out, void* k_cache, void* v_cache,
                             int n_q_heads, int n_kv_heads, int head_dim, int t_kv, const void* d_pos, float epsilon)
{
    if (head_dim != 128 || n_q_heads <= 0 || n_kv_heads <= 0 || t_kv <= 0 || !d_pos) { return -1; }
    if (!q || !k || !v || !cos_tab || !sin_tab || !q_out || !k_cache || !v_cache) { return -1; }
    if ((q_norm_w == nullptr) != (k_norm_w == nullptr)) { return -1; }          // both (Qwen3-style heads) or neither (Llama-style)
    qk_norm_rope_kv_kernel<<<n_q_heads + 2 * n_kv_heads, 64, 0, stream()>>>((const uint16_t*)q, (const uint16_t*)k, (const uint16_t*)v,
                                                                           (const uint16_t*)q_norm_w, (const uint16_t*)k_norm_w,
                                                                           (const uint16_t*)cos_tab, (const uint16_t*)sin_tab,
                                                                           (uint16_t*)q_out, (uint16_t*)k_cache, (uint16_t*)v_cache,
                                                                           n_q_heads, n_kv_heads, t_kv, (const int*)d_pos, epsilon);
    return finish("qk_norm_rope_kv");
}

namespace
{

struct AttentionWorkspace
{
    size_t scores, stats, partial, total;
    int n_blocks;
};

AttentionWorkspace attention_workspace(int n_q_heads, int t_kv)
{
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    AttentionWorkspace w{};
    w.n_blocks = (t_kv + ATT_KEYS - 1) / ATT_KEYS;
    w.scores = 0;
    w.stats = up(w.scores + (size_t)n_q_heads * t_kv * 2);
    w.partial = up(w.stats + (size_t)n_q_heads * w.n_blocks * sizeof(float2));
    w.total = up(w.partial + (size_t)w.n_blocks * n_q_heads * 128 * sizeof(float));
    return w;
}

template <int G>
void launch_attention(const uint16_t* q, const uint16_t* kc, const uint16_t* vc, uint16_t* y, char* ws, const AttentionWorkspace& w,
                      int n_q_heads, int n_kv_heads, int t_kv, const int* pos)
{
    const dim3 grid(w.n_blocks, n_kv_heads);
    uint16_t* scores = (uint16_t*)(ws + w.scores);
    float2* stats = (float2*)(ws + w.stats);
    float* partial = (float*)(ws + w.partial);
    attn_scores_kernel<G><<<grid, 256, 0, stream()>>>(q, kc, scores, stats, t_kv, w.n_blocks, pos, 1.0f / sqrtf(128.0f));
    attn_pv_kernel<G><<<grid, 256, 0, stream()>>>(scores, stats, vc, partial, t_kv, w.n_blocks, pos, n_q_heads);
    const int n_out = n_q_heads * 128;
    attn_combine_kernel<<<(n_out + 63) / 64, 256, 0, stream()>>>(partial, y, n_out, t_kv, pos);
}

}    // namespace

unsigned long long hip_attention_decode_workspace_bytes(int n_q_heads, int n_kv_heads, int t_kv)
{
    if (n_q_heads <= 0 || n_kv_heads <= 0 || t_kv <= 0) { return 0; }
    return attention_workspace(n_q_heads, t_kv).total;
}

int hip_attention_decode_bf16(const void* q, const void* k_cache, const void* v_cache, void* y, void* workspace, unsigned long long workspace_bytes,
                              int n_q_heads, int n_kv_heads, int head_dim, int t_kv, const void* d_pos)
{
    if (head_dim != 128 || n_kv_heads <= 0 || n_q_heads <= 0 || n_q_heads % n_kv_heads != 0 || t_kv <= 0 || !d_pos) { return -1; }
    if (!q || !k_cache || !v_cache || !y || !workspace || !aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(workspace)) { return -1; }
    const AttentionWorkspace w = attention_workspace(n_q_heads, t_kv);
    if (workspace_bytes < w.total) { return -1; }
    const uint16_t* qp = (const uint16_t*)q;
    const uint16_t* kc = (const uint16_t*)k_cache;
    const uint16_t* vc = (const uint16_t*)v_cache;
    const int* pos = (const int*)d_pos;
    switch (n_q_heads / n_kv_heads)
    {
    case 1: launch_attention<1>(qp, kc, vc, (uint16_t*)y, (char*)workspace, w, n_q_heads, n_kv_heads, t_kv, pos); break;
    case 2: launch_attention<2>(qp, kc, vc, (uint16_t*)y, (char*)workspace, w, n_q_heads, n_kv_heads, t_kv, pos); break;
    case 4: launch_attention<4>(qp, kc, vc, (uint16_t*)y, (char*)workspace, w, n_q_heads, n_kv_heads, t_kv, pos); break;
    default: return -1;
    }
    return finish("attention_decode");
}

int hip_attention_decode_fused_bf16(const void* q, const void* k, const void* v, const void* q_norm_w, const void* k_norm_w,
                                    const void* cos_tab, const void* sin_tab, void* k_cache, void* v_cache, void* y,
                                    void* workspace, unsigned long long workspace_bytes,
                                    int n_q_heads, int n_kv_heads, int head_dim, int t_kv, const void* d_pos, float epsilon)
{
    if (head_dim != 128 || n_kv_heads <= 0 || n_q_heads <= 0 || n_q_heads % n_kv_heads != 0 || t_kv <= 0 || !d_pos) { return -1; }
    if (!q || !k || !v || !cos_tab || !sin_tab || !k_cache || !v_cache || !y || !workspace) { return -1; }
    if ((q_norm_w == nullptr) != (k_norm_w == nullptr)) { return -1; }          // both (Qwen3-style heads) or neither (Llama-style)
    if (!aligned16(k_cache) || !aligned16(v_cache) || !aligned16(workspace)) { return -1; }
    const AttentionWorkspace w = attention_workspace(n_q_heads, t_kv);
    if (workspace_bytes < w.total || w.n_blocks > ATT_MAX_BLOCKS) { return -1; }
    const dim3 grid(w.n_blocks, n_kv_heads);
    float2* stats = (float2*)((char*)workspace + w.stats);
    float* partial = (float*)((char*)workspace + w.partial);
    const float scale = 1.0f / sqrtf(128.0f);
    const int* pos = (const int*)d_pos;
#define CCQ_ATTN_FUSED(G)                                                                                                                    \
    attn_fused_kernel<G><<<grid, 256, 0, stream()>>>((const uint16_t*)q, (const uint16_t*)k, (const uint16_t*)v, (const uint16_t*)q_norm_w, \
                                                     (const uint16_t*)k_norm_w, (const uint16_t*)cos_tab, (const uint16_t*)sin_tab,        \
                                                     (uint16_t*)k_cache, (uint16_t*)v_cache, stats, partial, t_kv, w.n_blocks, pos,        \
                                                     n_q_heads, epsilon, scale)
    switch (n_q_heads / n_kv_heads)
    {
    case 1: CCQ_ATTN_FUSED(1); break;
    case 2: CCQ_ATTN_FUSED(2); break;
    case 4: CCQ_ATTN_FUSED(4); break;
    default: return -1;
    }
#undef CCQ_ATTN_FUSED
    const int n_out = n_q_heads * 128;
    attn_rescale_combine_kernel<<<n_out / 64, 256, 0, stream()>>>(partial, stats, (uint16_t*)y, n_out, t_kv, w.n_blocks, pos);
    return finish("attention_decode_fused");
}

int hip_attention_decode_exact_bf16(const void* q, const void* k, const void* v, const void* q_norm_w, const void* k_norm_w,
                                    const void* cos_tab, const void* sin_tab, void* k_cache, void* v_cache, void* y,
                                    void* workspace, unsigned long long workspace_bytes,
                                    int n_q_heads, int n_kv_heads, int head_dim, int t_kv, const void* d_pos, float epsilon)
{
    if (head_dim != 128 || n_kv_heads <= 0 || n_q_heads <= 0 || n_q_heads % n_kv_heads != 0 || t_kv <= 0 || !d_pos) { return -1; }
    if (!q || !k || !v || !cos_tab || !sin_tab || !k_cache || !v_cache || !y || !workspace) { return -1; }
    if ((q_norm_w == nullptr) != (k_norm_w == nullptr)) { return -1; }
    if (!aligned16(k_cache) || !aligned16(v_cache) || !aligned16(workspace)) { return -1; }
    const AttentionWorkspace w = attention_workspace(n_q_heads, t_kv);
    if (workspace_bytes < w.total) { return -1; }
    const dim3 grid(w.n_blocks, n_kv_heads);
    uint16_t* scores = (uint16_t*)((char*)workspace + w.scores);
    float2* stats = (float2*)((char*)workspace + w.stats);
    float* partial = (float*)((char*)workspace + w.partial);
    const float scale = 1.0f / sqrtf(128.0f);
    const int* pos = (const int*)d_pos;
#define CCQ_ATTN_EXACT(G)                                                                                                                            \
    attn_fused_kernel<G, true><<<grid, 256, 0, stream()>>>((const uint16_t*)q, (const uint16_t*)k, (const uint16_t*)v, (const uint16_t*)q_norm_w,   \
                                                           (const uint16_t*)k_norm_w, (const uint16_t*)cos_tab, (const uint16_t*)sin_tab,          \
                                                           (uint16_t*)k_cache, (uint16_t*)v_cache, stats, partial, t_kv, w.n_blocks, pos,          \
                                                           n_q_heads, epsilon, scale, scores);                                                      \
    attn_pv_kernel<G><<<grid, 256, 0, stream()>>>(scores, stats, (const uint16_t*)v_cache, partial, t_kv, w.n_blocks, pos, n_q_heads)
    switch (n_q_heads / n_kv_heads)
    {
    case 1: CCQ_ATTN_EXACT(1); break;
    case 2: CCQ_ATTN_EXACT(2); break;
    case 4: CCQ_ATTN_EXACT(4); break;
    default: return -1;
    }
#undef CCQ_ATTN_EXACT
    const int n_out = n_q_heads * 128;
    attn_combine_kernel<<<(n_out + 63) / 64, 256, 0, stream()>>>(partial, (uint16_t*)y, n_out, t_kv, pos);
    return finish("attention_decode_exact");
}

// room for either use: the per-block candidates of hip_argmax_bf16, or the candidate list a linear launch leaves
unsigned long long hip_argmax_workspace_bytes(unsigned int n)
{
    const unsigned long long blocks = (n + ARGMAX_PER_BLOCK - 1) / ARGMAX_PER_BLOCK;
    const unsigned long long list = 16ull + ((unsigned long long)n / 2 + 16) * 8;
    return ((blocks * 8 > list ? blocks * 8 : list) + 255ull) & ~255ull;
}

int hip_argmax_pick_embed_bf16(const void* workspace, unsigned int n, void* d_index, void* d_pos, const void* embed_W, void* embed_y, int D, int n_rows)
{
    if (!workspace || !aligned16(workspace) || !d_index || n == 0) { return -1; }
    if (embed_W && (!embed_y || D <= 0 || D % 8 != 0 || n_rows <= 0 || !aligned16(embed_W) || !aligned16(embed_y))) { return -1; }
    const int blocks = embed_W ? (D / 8 + 255) / 256 : 1;
    argmax_pick_embed_kernel<<<blocks < 1 ? 1 : blocks, 256, 0, stream()>>>(workspace, n, (int*)d_index, (int*)d_pos, (const uint16_t*)embed_W, (uint16_t*)embed_y, D, n_rows);
    return finish("argmax_pick_embed");
}

int hip_argmax_bf16(const void* x, unsigned int n, void* d_index, void* d_pos, void* workspace)
{
    if (!x || !d_index || !workspace || n == 0) { return -1; }
    const unsigned blocks = (n + ARGMAX_PER_BLOCK - 1) / ARGMAX_PER_BLOCK;
    float* cand_v = (float*)workspace;
    unsigned* cand_i = (unsigned*)workspace + blocks;
    argmax_blocks_kernel<<<blocks, 256, 0, stream()>>>((const uint16_t*)x, n, cand_v, cand_i);
    argmax_pick_kernel<<<1, 256, 0, stream()>>>(cand_v, cand_i, blocks, (int*)d_index, (int*)d_pos);
    return finish("argmax_bf16");
}
