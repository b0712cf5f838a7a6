// C-ABI entry points of the prompt-phase neighbours (kernels in prefill_kernels.h).
#include "../../include/cccc_hip_quant.h"
#include "prefill_kernels.h"
#include "runtime.h"
#include <cmath>

using namespace ccq;

namespace
{
inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }
}    // namespace

int hip_qk_norm_rope_kv_rows_bf16(const void* q, const void* k, const void* v, const void* q_norm_w, const void* k_norm_w,
                                  const void* cos_tab, const void* sin_tab, void* q_out, void* k_cache, void* v_cache,
                                  int n_q_heads, int n_kv_heads, int head_dim, int t_kv, int n_tokens, int pos0, float epsilon)
{
    if (head_dim != 128 || n_q_heads <= 0 || n_kv_heads <= 0 || t_kv <= 0 || n_tokens <= 0 || n_tokens > 65535) { return -1; }
    if (pos0 < 0 || (long long)pos0 + n_tokens > t_kv) { return -1; }
    if (!q || !k || !v || !cos_tab || !sin_tab || !q_out || !k_cache || !v_cache) { return -1; }
    if ((q_norm_w == nullptr) != (k_norm_w == nullptr)) { return -1; }
    const dim3 grid((n_q_heads + 2 * n_kv_heads + 3) / 4, n_tokens);
    qk_norm_rope_kv_rows_kernel<<<grid, 256, 0, stream()>>>((const uint16_t*)q, (const uint16_t*)k, (const uint16_t*)v, (const uint16_t*)q_norm_w,
                                                           (const uint16_t*)k_norm_w, (const uint16_t*)cos_tab, (const uint16_t*)sin_tab,
                                                           (uint16_t*)q_out, (uint16_t*)k_cache, (uint16_t*)v_cache, n_q_heads, n_kv_heads, t_kv, pos0, epsilon);
    return finish("qk_norm_rope_kv_rows");
}

int hip_attention_prefill_bf16(const void* q, const void* k_cache, const void* v_cache, void* y,
                               int n_q_heads, int n_kv_heads, int head_dim, int t_kv, int n_tokens, int pos0)
{
    if (head_dim != 128 || n_kv_heads <= 0 || n_q_heads <= 0 || n_q_heads % n_kv_heads != 0 || t_kv <= 0 || n_tokens <= 0) { return -1; }
    if (pos0 < 0 || (long long)pos0 + n_tokens > t_kv || n_kv_heads > 65535) { return -1; }
    if (!q || !k_cache || !v_cache || !y || !aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache)) { return -1; }
    if ((long long)((n_tokens + 15) / 16) * n_kv_heads > 0x7FFFFFFFLL) { return -1; }
    // the kernel addresses cache rows with 32-bit byte offsets inside a KV head (row * 256)
    if ((long long)pos0 + n_tokens > (1LL << 24)) { return -1; }
    const dim3 grid((unsigned)((n_tokens + 15) / 16) * n_kv_heads);
    const float scale = 1.0f / sqrtf(128.0f);
#define CCQ_ATTN_PREFILL(G)                                                                                                                  \
    attn_prefill_kernel<G><<<grid, 256, 0, stream()>>>((const uint16_t*)q, (const uint16_t*)k_cache, (const uint16_t*)v_cache, (uint16_t*)y, \
                                                       n_q_heads, t_kv, n_tokens, pos0, scale)
    switch (n_q_heads / n_kv_heads)
    {
    case 1: CCQ_ATTN_PREFILL(1); break;
    case 2: CCQ_ATTN_PREFILL(2); break;
    case 4: CCQ_ATTN_PREFILL(4); break;
    default: return -1;
    }
#undef CCQ_ATTN_PREFILL
    return finish("attention_prefill");
}

int hip_add_bf16(const void* a, const void* b, void* y, unsigned long long n)
{
    if (!a || !b || !y || n == 0 || n % 8 != 0 || !aligned16(a) || !aligned16(b) || !aligned16(y)) { return -1; }
    const long long chunks = (long long)(n / 8);
    const long long blocks = (chunks + 255) / 256, cap = (long long)cu_count() * 16;
    add_rows_kernel<<<(unsigned)(blocks < cap ? blocks : cap), 256, 0, stream()>>>((const u32x4*)a, (const u32x4*)b, (u32x4*)y, chunks);
    return finish("add_bf16");
}

int hip_add_rms_norm_bf16(const void* a, const void* b, void* sum, const void* norm_w, void* y, unsigned int rows, unsigned int inner, float epsilon)
{
    if (!a || !b || !sum || !norm_w || !y || rows == 0 || inner == 0 || inner % 8 != 0 || inner > 64u * 8u * RMS_CHUNKS) { return -1; }
    if (!aligned16(a) || !aligned16(b) || !aligned16(sum) || !aligned16(norm_w) || !aligned16(y)) { return -1; }
    add_rms_norm_rows_kernel<<<(rows + 3) / 4, 256, 0, stream()>>>((const uint16_t*)a, (const uint16_t*)b, (uint16_t*)sum, (const uint16_t*)norm_w,
                                                                   (uint16_t*)y, rows, inner, epsilon);
    return finish("add_rms_norm_bf16");
}

int hip_swiglu_bf16(const void* gate, const void* up, void* y, unsigned long long n)
{
    if (!gate || !up || !y || n == 0 || n % 8 != 0 || !aligned16(gate) || !aligned16(up) || !aligned16(y)) { return -1; }
    const long long chunks = (long long)(n / 8);
    const long long blocks = (chunks + 255) / 256, cap = (long long)cu_count() * 16;
    swiglu_rows_kernel<<<(unsigned)(blocks < cap ? blocks : cap), 256, 0, stream()>>>((const u32x4*)gate, (const u32x4*)up, (u32x4*)y, chunks);
    return finish("swiglu_bf16");
}
