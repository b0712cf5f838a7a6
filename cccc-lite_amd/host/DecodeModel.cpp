#include "DecodeModel.h"
#include "../../include/cccc_hip_quant.h"
#include <hip/hip_runtime.h>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <vector>

namespace cccc
{

static std::unique_ptr<Matrix> make(int w, int h, DataType dt, GpuControl* gpu) { return std::make_unique<Matrix>(w, h, 1, 1, dt, gpu); }

static void zero(Matrix& m, size_t bytes) { (void)hipMemset(m.data(), 0, bytes); }

DecodeModel::DecodeModel(const DecodeConfig& cfg, GpuControl* gpu) : cfg_(cfg), gpu_(gpu)
{
    gpu_->setAsCurrent();
    const int q_out = cfg.n_q * cfg.head_dim, kv_out = cfg.n_kv * cfg.head_dim;
    layers_.resize(cfg.layers);
    for (auto& L : layers_)
    {
        // linears are allocated as 1-byte tensors and re-typed by loadQuantizedDirect; (W, H) = (in, out)
        L.rms_attn = make(cfg.hidden, 1, BFLOAT16, gpu);
        L.wq = make(cfg.hidden, q_out, FP8_E5M2, gpu);
        L.wk = make(cfg.hidden, kv_out, FP8_E5M2, gpu);
        L.wv = make(cfg.hidden, kv_out, FP8_E5M2, gpu);
        L.q_norm = make(cfg.head_dim, 1, BFLOAT16, gpu);
        L.k_norm = make(cfg.head_dim, 1, BFLOAT16, gpu);
        L.wo = make(q_out, cfg.hidden, FP8_E5M2, gpu);
        L.rms_ffn = make(cfg.hidden, 1, BFLOAT16, gpu);
        L.w_gate = make(cfg.hidden, cfg.inter, FP8_E5M2, gpu);
        L.w_up = make(cfg.hidden, cfg.inter, FP8_E5M2, gpu);
        L.w_down = make(cfg.inter, cfg.hidden, FP8_E5M2, gpu);
        k_cache_.push_back(std::make_unique<Matrix>(cfg.head_dim, cfg.t_kv, 1, cfg.n_kv, BFLOAT16, gpu));
        v_cache_.push_back(std::make_unique<Matrix>(cfg.head_dim, cfg.t_kv, 1, cfg.n_kv, BFLOAT16, gpu));
        const size_t cache_bytes = (size_t)cfg.head_dim * cfg.t_kv * cfg.n_kv * 2;
        zero(*k_cache_.back(), cache_bytes);
        zero(*v_cache_.back(), cache_bytes);
    }
    emb_ = make(cfg.hidden, cfg.vocab, BFLOAT16, gpu);
    rms_final_ = make(cfg.hidden, 1, BFLOAT16, gpu);
    lm_head_ = make(cfg.hidden, cfg.vocab, FP8_E5M2, gpu);
    logits_ = make(cfg.vocab, 1, BFLOAT16, gpu);
    x_ = make(cfg.hidden, 1, BFLOAT16, gpu);
    r1_ = make(cfg.hidden, 1, BFLOAT16, gpu);
    q_ = make(q_out, 1, BFLOAT16, gpu);
    k_ = make(kv_out, 1, BFLOAT16, gpu);
    v_ = make(kv_out, 1, BFLOAT16, gpu);
    att_ = make(q_out, 1, BFLOAT16, gpu);
    gated_ = make(cfg.inter, 1, BFLOAT16, gpu);
    attn_ws_bytes_ = hip_attention_decode_workspace_bytes(cfg.n_q, cfg.n_kv, cfg.t_kv);
    attn_ws_ = make((int)((attn_ws_bytes_ + 3) / 4), 1, FLOAT, gpu);
    argmax_ws_ = make((int)((hip_argmax_workspace_bytes((unsigned)cfg.vocab) + 3) / 4), 1, FLOAT, gpu);

    // RoPE tables as the reference's graph builds them (cccc/NetCifa.cpp:431-475): float math on the host,
    // stored to BF16 by truncation (cccc/types.h:43-48)
    const int half = cfg.head_dim / 2;
    std::vector<uint16_t> cos_h((size_t)cfg.t_kv * half), sin_h(cos_h.size());
    for (int t = 0; t < cfg.t_kv; t++)
    {
        for (int d = 0; d < half; d++)
        {
            const float angle = t * std::pow(cfg.theta, -2.0f * d / cfg.head_dim);
            const float c = (float)std::cos(angle), s = (float)std::sin(angle);
            uint32_t cu, su;
            std::memcpy(&cu, &c, 4);
            std::memcpy(&su, &s, 4);
            cos_h[(size_t)t * half + d] = (uint16_t)(cu >> 16);
            sin_h[(size_t)t * half + d] = (uint16_t)(su >> 16);
        }
    }
    cos_ = make(half, cfg.t_kv, BFLOAT16, gpu);
    sin_ = make(half, cfg.t_kv, BFLOAT16, gpu);
    cos_->copyFromHost(cos_h.data(), cos_h.size() * 2);
    sin_->copyFromHost(sin_h.data(), sin_h.size() * 2);

    void* p = nullptr;
    gpu_->malloc(&p, 2 * sizeof(int));
    d_state_ = (int*)p;
    (void)hipMemset(d_state_, 0, 2 * sizeof(int));
}

DecodeModel::~DecodeModel()
{
    if (d_state_) { gpu_->free(d_state_); }
}

Matrix* DecodeModel::tensor(int layer, int which)
{
    if (which >= EMB)
    {
        return which == EMB ? emb_.get() : which == RMS_FINAL ? rms_final_.get() : which == LM_HEAD ? lm_head_.get() : nullptr;
    }
    if (layer < 0 || layer >= cfg_.layers) { return nullptr; }
    Layer& L = layers_[layer];
    Matrix* table[] = { L.rms_attn.get(), L.wq.get(), L.wk.get(), L.wv.get(), L.q_norm.get(), L.k_norm.get(), L.wo.get(),
                        L.rms_ffn.get(), L.w_gate.get(), L.w_up.get(), L.w_down.get() };
    return (which >= 0 && which <= W_DOWN) ? table[which] : nullptr;
}

int DecodeModel::setBlockScales(int layer, int which, const void* host, size_t n_scales)
{
    Matrix* m = tensor(layer, which);
    if (!m || m->getDataType() != FP4_E2M1 || (int64_t)n_scales != (m->getDataSize() + Matrix::fp4BlockSize() - 1) / Matrix::fp4BlockSize()) { return -1; }
    m->setBlockScaleFromHost(host, (int64_t)n_scales);
    return m->getBlockScaleData() ? 0 : 1;
}

Matrix* DecodeModel::activation(int which)
{
    Matrix* table[] = { x_.get(), r1_.get(), q_.get(), k_.get(), v_.get(), att_.get(), gated_.get() };
    return (which >= 0 && which <= ACT_GATED) ? table[which] : nullptr;
}

int DecodeModel::setTensor(int layer, int which, const void* host, size_t bytes, DataType dt, float scale)
{
    Matrix* m = tensor(layer, which);
    if (!m) { return -1; }
    if (Rocblas::isQuantized(dt))
    {
        if ((int64_t)bytes != (dt == FP4_E2M1 ? (m->getDataSize() + 1) / 2 : m->getDataSize())) { return -1; }
        // only a tall FP8 weight (lm_head) is read through its tiled copy by the fused decode kernels
        m->setAllowRepack(repack_linears_ || (which == LM_HEAD && dt != FP4_E2M1));
        m->loadQuantizedDirect((const uint8_t*)host, (int64_t)bytes, scale, dt);
        return 0;
    }
    return m->copyFromHost(host, bytes);
}

int DecodeModel::quantizeLinear(int layer, int which, const void* device_bf16, DataType to)
{
    const bool linear = which == WQ || which == WK || which == WV || which == WO || which == W_GATE || which == W_UP || which == W_DOWN ||
                        (which == LM_HEAD && !tied_lm_head_);
    Matrix* m = tensor(layer, which);
    if (!m || !linear || !device_bf16 || !Rocblas::isQuantized(to)) { return -1; }
    gpu_->setAsCurrent();
    Matrix tmp(m->getWidth(), m->getHeight(), 1, 1, BFLOAT16, gpu_);
    // only a tall FP8 weight (lm_head) is read through its tiled copy by the fused decode kernels
    tmp.setAllowRepack(repack_linears_ || (which == LM_HEAD && to != FP4_E2M1));
    if (GpuControl::copyDeviceToDevice(tmp.data(), device_bf16, (size_t)tmp.getDataSize() * 2) != 0) { return 1; }
    tmp.quantizeWeights(to);
    if (!Rocblas::isQuantized(tmp.getDataType())) { return -3; }
    *m = tmp;
    return 0;
}

int DecodeModel::loadNamedWeights(const WeightFile& file, DataType quantize_to, std::string* failed)
{
    gpu_->setAsCurrent();
    auto fail = [&](const std::string& name, int code) {
        if (failed) { *failed = name; }
        return code;
    };
    // norms and the embedding: BF16 tensors
    auto load_plain = [&](Matrix& m, const std::string& name) -> int {
        const auto wk = file.resolve(name);
        if (!wk.valid()) { return fail(name, -1); }
        if (wk.is_quant) { return fail(name, -3); }
        const std::vector<int> dim = { m.getWidth(), m.getHeight(), m.getChannel(), m.getNumber() };
        Matrix tmp(dim, BFLOAT16, gpu_);
        if (file.loadNamed(tmp, name) != 0) { return fail(name, -2); }
        if (tmp.getDataType() == FLOAT || tmp.getDataType() == HALF)      // the file's type was kept: round to BF16 on the device
        {
            Matrix bf(dim, BFLOAT16, gpu_);
            if (hip_convert(tmp.data(), (int)tmp.getDataType(), bf.data(), (int)BFLOAT16, (unsigned)tmp.getDataSize(), 1.0f) != 0) { return fail(name, -3); }
            (void)hipDeviceSynchronize();
            tmp = bf;
        }
        if (tmp.getDataType() != BFLOAT16) { return fail(name, -3); }
        m = tmp;
        return 0;
    };
    auto load_linear = [&](Matrix& m, const std::string& name, bool head = false) -> int {
        const bool tiled = head || repack_linears_;
        const auto wk = file.resolve(name);
        if (!wk.valid()) { return fail(name, -1); }
        if (wk.is_quant)
        {
            m.setAllowRepack(repack_linears_ || (tiled && wk.dt != FP4_E2M1));      // the fused FP4 kernels read the file layout only
            if (file.loadNamed(m, name) != 0) { return fail(name, -2); }
            if (wk.dt == FP4_E2M1 && !m.getBlockScaleData()) { return fail(name, -3); }    // FP4 without blockscale_<name>: no fused kernel
            return 0;
        }
        const bool tiled_q = repack_linears_ || (tiled && quantize_to != FP4_E2M1);
        Matrix tmp(m.getWidth(), m.getHeight(), 1, 1, BFLOAT16, gpu_);
        tmp.setAllowRepack(tiled_q);
        if (file.loadNamed(tmp, name) != 0) { return fail(name, -2); }
        if (tmp.getDataType() == FLOAT)
        {
            Matrix bf(m.getWidth(), m.getHeight(), 1, 1, BFLOAT16, gpu_);
            bf.setAllowRepack(tiled_q);
            if (hip_convert(tmp.data(), (int)FLOAT, bf.data(), (int)BFLOAT16, (unsigned)tmp.getDataSize(), 1.0f) != 0) { return fail(name, -3); }
            (void)hipDeviceSynchronize();
            tmp = bf;
        }
        tmp.quantizeWeights(quantize_to);
        if (!Rocblas::isQuantized(tmp.getDataType())) { return fail(name, -3); }
        m = tmp;
        return 0;
    };
    // a file without per-head norm weights is a model without them (scripts/convert_weights.py:231-239 decides the same way)
    qk_norm_ = cfg_.layers == 0 || file.resolve("W_qnorm_0").valid() || file.resolve("W_knorm_0").valid();
    int rc = load_plain(*emb_, "W_emb");
    if (rc == 0) { rc = load_plain(*rms_final_, "W_rms_final"); }
    // no W_lm_head entry: tied embeddings -- the head multiplies by the embedding table, which the reference never quantizes
    // (cccc/Net.cpp:1158-1190 skips EMBED tables and every view that shares their storage)
    setTiedLmHead(!file.resolve("W_lm_head").valid());
    if (rc == 0 && !tied_lm_head_) { rc = load_linear(*lm_head_, "W_lm_head", true); }
    for (int i = 0; i < cfg_.layers && rc == 0; i++)
    {
        Layer& L = layers_[i];
        const std::string n = std::to_string(i);
        const std::pair<Matrix*, const char*> plain[] = { { L.rms_attn.get(), "W_rms_attn_" }, { L.q_norm.get(), "W_qnorm_" }, { L.k_norm.get(), "W_knorm_" }, { L.rms_ffn.get(), "W_rms_ffn_" } };
        const std::pair<Matrix*, const char*> linear[] = { { L.wq.get(), "W_q_" }, { L.wk.get(), "W_k_" }, { L.wv.get(), "W_v_" }, { L.wo.get(), "W_o_" },
                                                          { L.w_gate.get(), "W_gate_" }, { L.w_up.get(), "W_up_" }, { L.w_down.get(), "W_down_" } };
        for (auto& [m, prefix] : plain)
        {
            const bool head_norm = m == L.q_norm.get() || m == L.k_norm.get();
            if (rc == 0 && (qk_norm_ || !head_norm)) { rc = load_plain(*m, prefix + n); }
        }
        for (auto& [m, prefix] : linear) { if (rc == 0) { rc = load_linear(*m, prefix + n); } }
    }
    return rc;
}

int DecodeModel::saveNamedWeights(const std::string& filename)
{
    gpu_->setAsCurrent();
    if (filename.empty() || hipDeviceSynchronize() != hipSuccess) { return -1; }
    WeightFileWriter w;
    // header: the first quantized tensor's type, else the first tensor's (cccc/Net.cpp:1243-1271)
    const DataType head = (!tied_lm_head_ && Rocblas::isQuantized(lm_head_->getDataType())) || layers_.empty() ? lm_head_->getDataType() : layers_[0].wq->getDataType();
    const char* names[] = { "auto", "float", "double", "half", "bfloat16", "fp8_e4m3", "fp8_e5m2", "fp4_e2m1" };
    const DataType order[] = { CURRENT, FLOAT, DOUBLE, HALF, BFLOAT16, FP8_E4M3, FP8_E5M2, FP4_E2M1 };
    std::string head_name = "auto";
    for (int i = 0; i < 8; i++) { if (order[i] == head) { head_name = names[i]; } }
    w.set_value("data_type", head_name);
    w.set_value("named_weights", std::string("1"));
    addNamedWeight(w, "W_emb", *emb_);
    addNamedWeight(w, "W_rms_final", *rms_final_);
    if (!tied_lm_head_) { addNamedWeight(w, "W_lm_head", *lm_head_); }
    for (int i = 0; i < cfg_.layers; i++)
    {
        Layer& L = layers_[i];
        const std::string n = std::to_string(i);
        const std::pair<Matrix*, const char*> tensors[] = {
            { L.rms_attn.get(), "W_rms_attn_" }, { L.wq.get(), "W_q_" }, { L.wk.get(), "W_k_" }, { L.wv.get(), "W_v_" },
            { L.q_norm.get(), "W_qnorm_" }, { L.k_norm.get(), "W_knorm_" }, { L.wo.get(), "W_o_" }, { L.rms_ffn.get(), "W_rms_ffn_" },
            { L.w_gate.get(), "W_gate_" }, { L.w_up.get(), "W_up_" }, { L.w_down.get(), "W_down_" } };
        for (auto& [m, prefix] : tensors)
        {
            if (!qk_norm_ && (m == L.q_norm.get() || m == L.k_norm.get())) { continue; }
            addNamedWeight(w, prefix + n, *m);
        }
    }
    return w.save(filename) > 0 ? 0 : -1;
}

void DecodeModel::setTiedLmHead(bool tied)
{
    if (tied == tied_lm_head_) { return; }
    tied_lm_head_ = tied;
    // the separate head's storage is only held while it is used
    if (tied) { lm_head_ = std::make_unique<Matrix>(cfg_.hidden, 1, 1, 1, FP8_E5M2, gpu_); }
    else { lm_head_ = std::make_unique<Matrix>(cfg_.hidden, cfg_.vocab, 1, 1, FP8_E5M2, gpu_); }
}

size_t DecodeModel::weightBytes() const
{
    const size_t q_out = (size_t)cfg_.n_q * cfg_.head_dim, kv_out = (size_t)cfg_.n_kv * cfg_.head_dim;
    const size_t per_layer = (size_t)cfg_.hidden * (q_out + 2 * kv_out) + q_out * cfg_.hidden + 3 * (size_t)cfg_.hidden * cfg_.inter;
    return per_layer * cfg_.layers + (size_t)cfg_.hidden * cfg_.vocab;
}

int DecodeModel::reset(int token, int pos)
{
    const int state[2] = { token, pos };
    if (GpuControl::copyHostToDevice(d_state_, state, sizeof(state)) != 0) { return 1; }
    // a step starts from the embedding of its token: the previous step's greedy pick leaves it behind, a reset fetches it
    return hip_embed_token_bf16(d_state_, emb_->data(), x_->data(), cfg_.hidden, cfg_.vocab);
}

int DecodeModel::currentToken()
{
    int t = -1;
    GpuControl::copyDeviceToHost(&t, d_state_, sizeof(int));
    return t;
}

int DecodeModel::currentPos()
{
    int p = -1;
    GpuControl::copyDeviceToHost(&p, d_state_ + 1, sizeof(int));
    return p;
}

static hip_fused_linear linear_desc(const Matrix& W, int n_out, int K, const void* x, void* y)
{
    hip_fused_linear d{};
    d.w_type = (int)W.getDataType();
    d.K = K;
    d.n_segments = 1;
    d.W[0] = W.data();
    d.n_out[0] = n_out;
    d.w_scale[0] = W.getQuantScale();
    d.blk_sc[0] = W.getBlockScaleData();
    d.block_size = Matrix::fp4BlockSize();
    d.Y[0] = y;
    d.X = x;
    return d;
}

int DecodeModel::step()
{
    const DecodeConfig& c = cfg_;
    const int q_out = c.n_q * c.head_dim, kv_out = c.n_kv * c.head_dim;
    const int* d_pos = d_state_ + 1;
    int rc = 0;
    for (int li = 0; li < c.layers && rc == 0; li++)
    {
        Layer& L = layers_[li];
        // 1. q, k, v = W_{q,k,v} rmsnorm(x): one launch, three weight segments
        // (a descriptor carries one weight type: projections stored in different FP8 formats go out as three launches)
        hip_fused_linear qkv = linear_desc(*L.wq, q_out, c.hidden, x_->data(), q_->data());
        qkv.norm_weight = L.rms_attn->data();
        qkv.norm_eps = c.eps;
        if (L.wk->getDataType() == L.wq->getDataType() && L.wv->getDataType() == L.wq->getDataType())
        {
            qkv.n_segments = 3;
            qkv.W[1] = L.wk->data(); qkv.n_out[1] = kv_out; qkv.w_scale[1] = L.wk->getQuantScale(); qkv.Y[1] = k_->data();
            qkv.W[2] = L.wv->data(); qkv.n_out[2] = kv_out; qkv.w_scale[2] = L.wv->getQuantScale(); qkv.Y[2] = v_->data();
            qkv.blk_sc[1] = L.wk->getBlockScaleData();
            qkv.blk_sc[2] = L.wv->getBlockScaleData();
            rc = hip_quant_linear_fused(&qkv);
        }
        else
        {
            rc = hip_quant_linear_fused(&qkv);
            for (Matrix* w : { L.wk.get(), L.wv.get() })
            {
                if (rc != 0) { break; }
                hip_fused_linear kv = linear_desc(*w, kv_out, c.hidden, x_->data(), w == L.wk.get() ? k_->data() : v_->data());
                kv.norm_weight = L.rms_attn->data();
                kv.norm_eps = c.eps;
                rc = hip_quant_linear_fused(&kv);
            }
        }
        // 2-3. per-head q/k norm (models that have one), RoPE, KV append and attention over the cache
        const void* q_norm_w = qk_norm_ ? L.q_norm->data() : nullptr;
        const void* k_norm_w = qk_norm_ ? L.k_norm->data() : nullptr;
        if (rc == 0 && !exact_attention_)
        {
            rc = hip_attention_decode_fused_bf16(q_->data(), k_->data(), v_->data(), q_norm_w, k_norm_w, cos_->data(), sin_->data(),
                                                 k_cache_[li]->data(), v_cache_[li]->data(), att_->data(), attn_ws_->data(), attn_ws_bytes_,
                                                 c.n_q, c.n_kv, c.head_dim, c.t_kv, d_pos, c.eps);
        }
        else if (rc == 0)
        {
            rc = hip_attention_decode_exact_bf16(q_->data(), k_->data(), v_->data(), q_norm_w, k_norm_w, cos_->data(), sin_->data(),
                                                 k_cache_[li]->data(), v_cache_[li]->data(), att_->data(), attn_ws_->data(), attn_ws_bytes_,
                                                 c.n_q, c.n_kv, c.head_dim, c.t_kv, d_pos, c.eps);
        }
        // 4. r1 = x + W_o att
        if (rc == 0)
        {
            hip_fused_linear o = linear_desc(*L.wo, c.hidden, q_out, att_->data(), r1_->data());
            o.residual = x_->data();
            rc = hip_quant_linear_fused(&o);
        }
        // 5. gated = silu(W_gate n) * (W_up n), n = rmsnorm(r1)
        if (rc == 0 && L.w_up->getDataType() != L.w_gate->getDataType())
        {
            // the SwiGLU pair kernel decodes both weights with one format: two formats go out as two linears (each with the
            // norm in front) and the product as a launch of its own, with the same roundings
            if (!gate_) { gate_ = make(c.inter, 1, BFLOAT16, gpu_); up_ = make(c.inter, 1, BFLOAT16, gpu_); }
            for (Matrix* w : { L.w_gate.get(), L.w_up.get() })
            {
                if (rc != 0) { break; }
                hip_fused_linear one = linear_desc(*w, c.inter, c.hidden, r1_->data(), w == L.w_gate.get() ? gate_->data() : up_->data());
                one.norm_weight = L.rms_ffn->data();
                one.norm_eps = c.eps;
                rc = hip_quant_linear_fused(&one);
            }
            if (rc == 0) { rc = hip_swiglu_bf16(gate_->data(), up_->data(), gated_->data(), (unsigned long long)c.inter); }
        }
        else if (rc == 0)
        {
            hip_fused_linear gu = linear_desc(*L.w_gate, c.inter, c.hidden, r1_->data(), gated_->data());
            gu.n_segments = 2;
            gu.pair = 1;
            gu.W[1] = L.w_up->data(); gu.n_out[1] = c.inter; gu.w_scale[1] = L.w_up->getQuantScale();
            gu.blk_sc[1] = L.w_up->getBlockScaleData();
            gu.norm_weight = L.rms_ffn->data();
            gu.norm_eps = c.eps;
            rc = hip_quant_linear_fused(&gu);
        }
        // 6. x = r1 + W_down gated
        if (rc == 0)
        {
            hip_fused_linear dn = linear_desc(*L.w_down, c.hidden, c.inter, gated_->data(), x_->data());
            dn.residual = r1_->data();
            rc = hip_quant_linear_fused(&dn);
        }
    }
    return rc == 0 ? head() : rc;
}

int DecodeModel::head()
{
    const DecodeConfig& c = cfg_;
    hip_fused_linear head = linear_desc(tied_lm_head_ ? *emb_ : *lm_head_, c.vocab, c.hidden, x_->data(), logits_->data());
    head.norm_weight = rms_final_->data();
    head.norm_eps = c.eps;
    head.argmax_workspace = argmax_ws_->data();            // the launch leaves the greedy candidates of its logits
    int rc = hip_quant_linear_fused(&head);
    // pick, advance the position, and fetch the next step's embedding row: one launch
    if (rc == 0) { rc = hip_argmax_pick_embed_bf16(argmax_ws_->data(), (unsigned)c.vocab, d_state_, d_state_ + 1, emb_->data(), x_->data(), c.hidden, c.vocab); }
    return rc;
}

int DecodeModel::prefill(const int* tokens, int n_tokens, int pos0)
{
    constexpr int kPiece = 2048;
    if (!tokens || n_tokens <= 0 || pos0 < 0 || (long long)pos0 + n_tokens > cfg_.t_kv) { return -1; }
    for (int i = 0; i < n_tokens; i++)
    {
        if (tokens[i] < 0 || tokens[i] >= cfg_.vocab) { return -1; }
    }
    gpu_->setAsCurrent();
    int rc = 0;
    for (int t0 = 0; t0 < n_tokens && rc == 0; t0 += kPiece)
    {
        const int n = n_tokens - t0 < kPiece ? n_tokens - t0 : kPiece;
        rc = prefillPiece(tokens + t0, n, pos0 + t0, t0 + n == n_tokens);
    }
    return rc;
}

int DecodeModel::prefillPiece(const int* tokens, int n, int pos0, bool last)
{
    const DecodeConfig& c = cfg_;
    const int q_out = c.n_q * c.head_dim, kv_out = c.n_kv * c.head_dim;
    if (pf_.tokens < n)
    {
        pf_.tokens = n;
        pf_.ids = make(n, 1, FLOAT, gpu_);
        for (auto* m : { &pf_.x, &pf_.xn, &pf_.o, &pf_.r1 }) { *m = make(c.hidden, n, BFLOAT16, gpu_); }
        for (auto* m : { &pf_.q, &pf_.q_rot, &pf_.att }) { *m = make(q_out, n, BFLOAT16, gpu_); }
        for (auto* m : { &pf_.k, &pf_.v }) { *m = make(kv_out, n, BFLOAT16, gpu_); }
        for (auto* m : { &pf_.gate, &pf_.up, &pf_.gated }) { *m = make(c.inter, n, BFLOAT16, gpu_); }
    }
    // Every kernel of the piece goes to the library's stream of this thread.  The host copies below are the mirror's blocking
    // copies, which wait for that stream first (GpuControl::copyHostToDevice): nothing an earlier launch still reads
    // (pf_.ids, the step state) is overwritten under it, and a copy has landed before anything is launched behind it.
    const hipStream_t stream = (hipStream_t)hip_quant_get_stream();
    std::vector<float> ids(tokens, tokens + n);
    if (GpuControl::copyHostToDevice(pf_.ids->data(), ids.data(), (size_t)n * sizeof(float)) != 0) { return 1; }
    int rc = hip_embed_fwd((int)BFLOAT16, pf_.ids->data(), emb_->data(), pf_.x->data(), c.hidden, n, 1);
    // y [n][n_out] = x [n][K] W^T: the weight is the A operand, transposed, as cccc's batchedMul passes it (scripts/convert_weights.py:492)
    auto linear = [&](const Matrix& W, int n_out, int K, const Matrix& x, Matrix& y) {
        return gpu_->rocblas_->gemm(MATRIX_TRANS, MATRIX_NO_TRANS, n_out, n, K, 1.0f, W.data(), W.getDataType(), K, W.getQuantScale(),
                                    x.data(), BFLOAT16, K, 1.0f, 0.0f, y.data(), BFLOAT16, n_out, 0.0f,
                                    W.getDataType() == FP4_E2M1 ? (const uint8_t*)W.getBlockScaleData() : nullptr, nullptr);
    };
    auto norm = [&](Matrix& x, Matrix& y, Matrix& w) {
        return hip_rms_norm_fwd((int)BFLOAT16, x.data(), y.data(), w.data(), nullptr, (unsigned)n, (unsigned)c.hidden, c.eps);
    };
    // a residual add and the norm behind it go out as one launch where the row fits the kernel (hidden <= 4096)
    const bool fused_norm = c.hidden % 8 == 0 && c.hidden <= 4096;
    auto add_norm = [&](Matrix& a, Matrix& b, Matrix& sum, Matrix& w, Matrix& y) {
        if (fused_norm) { return hip_add_rms_norm_bf16(a.data(), b.data(), sum.data(), w.data(), y.data(), (unsigned)n, (unsigned)c.hidden, c.eps); }
        const int r = hip_add_bf16(a.data(), b.data(), sum.data(), (unsigned long long)n * c.hidden);
        return r != 0 ? r : norm(sum, y, w);
    };
    // The fused GEMM launches below are matrix-matrix kernels; up to 16 tokens the separate calls run the matrix-vector
    // kernels, which stay ahead on tiled copies (16 tokens: 3.3 ms either way, 2 tokens 2.8 against 3.1) but not on the file
    // layout from about 5 tokens on (16 tokens: 4.1 -> 3.7 ms of a 36-layer 4096-wide model, 6 tokens 3.9 -> 3.5)
    // FP4 linears reach the register-fed GEMM and its fused launches only through their tiled copies (codes and scales in
    // matrix-core operand order; the two-operand kernel on the file layout runs at half the rate).  A model loaded without
    // them builds them when a prompt of 17 tokens or more first needs them: 1.125x the FP4 weight memory from then on.
    if (n >= 17)
    {
        for (auto& L : layers_)
        {
            for (Matrix* w : { L.wq.get(), L.wk.get(), L.wv.get(), L.wo.get(), L.w_gate.get(), L.w_up.get(), L.w_down.get() })
            {
                if (w->getDataType() == FP4_E2M1 && !w->hasTiled() && w->getWidth() % 128 == 0)
                {
                    w->setAllowRepack(true);
                    w->prepareTiled();
                }
            }
        }
    }
    const bool fuse_gemms = n >= (c.layers > 0 && layers_[0].wq->hasTiled() ? 17 : 5);
    // sum = res + W x and y = norm(sum): where the GEMM splits its k range the launch that adds the partial sums does the add
    // and the norm as well (-1: this shape does not split, or the library has no such kernel for it)
    auto linear_add_norm = [&](const Matrix& W, int n_out, int K, const Matrix& x, Matrix& res, Matrix& sum, Matrix& w, Matrix& y) {
        int r = !fuse_gemms ? -1 : hip_quant_gemm_add_rms_norm(n_out, n, K, W.data(), (int)W.getDataType(), K, W.getQuantScale(), x.data(), K,
                                                               res.data(), sum.data(), w.data(), y.data(), c.eps);
        if (r >= 0) { return r; }
        r = linear(W, n_out, K, x, *pf_.o);
        return r != 0 ? r : add_norm(res, *pf_.o, sum, w, y);
    };
    if (rc == 0 && c.layers > 0) { rc = norm(*pf_.x, *pf_.xn, *layers_[0].rms_attn); }
    for (int li = 0; li < c.layers && rc == 0; li++)
    {
        Layer& L = layers_[li];
        // q, k, v: one launch for three weights of one type, else three calls
        int qkv = -1;
        if (rc == 0 && fuse_gemms && L.wk->getDataType() == L.wq->getDataType() && L.wv->getDataType() == L.wq->getDataType())
        {
            const int widths[3] = { q_out, kv_out, kv_out };
            const void* const weights[3] = { L.wq->data(), L.wk->data(), L.wv->data() };
            const float scales[3] = { L.wq->getQuantScale(), L.wk->getQuantScale(), L.wv->getQuantScale() };
            void* const outputs[3] = { pf_.q->data(), pf_.k->data(), pf_.v->data() };
            qkv = hip_quant_gemm_segments(3, widths, weights, scales, outputs, widths, (int)L.wq->getDataType(), n, c.hidden, c.hidden, pf_.xn->data(), c.hidden);
            if (qkv > 0) { rc = qkv; }
        }
        if (qkv < 0)
        {
            if (rc == 0) { rc = linear(*L.wq, q_out, c.hidden, *pf_.xn, *pf_.q); }
            if (rc == 0) { rc = linear(*L.wk, kv_out, c.hidden, *pf_.xn, *pf_.k); }
            if (rc == 0) { rc = linear(*L.wv, kv_out, c.hidden, *pf_.xn, *pf_.v); }
        }
        if (rc == 0)
        {
            rc = hip_qk_norm_rope_kv_rows_bf16(pf_.q->data(), pf_.k->data(), pf_.v->data(), qk_norm_ ? L.q_norm->data() : nullptr,
                                               qk_norm_ ? L.k_norm->data() : nullptr, cos_->data(), sin_->data(), pf_.q_rot->data(),
                                               k_cache_[li]->data(), v_cache_[li]->data(), c.n_q, c.n_kv, c.head_dim, c.t_kv, n, pos0, c.eps);
        }
        if (rc == 0)
        {
            rc = hip_attention_prefill_bf16(pf_.q_rot->data(), k_cache_[li]->data(), v_cache_[li]->data(), pf_.att->data(),
                                            c.n_q, c.n_kv, c.head_dim, c.t_kv, n, pos0);
        }
        // o, the residual add and the norm behind it: one call where the GEMM splits its k range (short prompts), else two
        if (rc == 0) { rc = linear_add_norm(*L.wo, c.hidden, q_out, *pf_.att, *pf_.x, *pf_.r1, *L.rms_ffn, *pf_.xn); }
        // gate, up and their SwiGLU product: one launch for two weights of one type, else the three calls
        int fused = -1;
        if (rc == 0 && fuse_gemms && L.w_gate->getDataType() == L.w_up->getDataType())
        {
            fused = hip_quant_gemm_swiglu(c.inter, n, c.hidden, L.w_gate->data(), L.w_up->data(), (int)L.w_gate->getDataType(), c.hidden,
                                          L.w_gate->getQuantScale(), L.w_up->getQuantScale(), pf_.xn->data(), c.hidden, pf_.gated->data(), c.inter);
            if (fused > 0) { rc = fused; }
        }
        if (fused < 0)
        {
            if (rc == 0) { rc = linear(*L.w_gate, c.inter, c.hidden, *pf_.xn, *pf_.gate); }
            if (rc == 0) { rc = linear(*L.w_up, c.inter, c.hidden, *pf_.xn, *pf_.up); }
            if (rc == 0) { rc = hip_swiglu_bf16(pf_.gate->data(), pf_.up->data(), pf_.gated->data(), (unsigned long long)n * c.inter); }
        }
        // x = r1 + ffn, and the next layer's first norm with it (the head normalises the last token's row itself)
        if (rc == 0 && li + 1 < c.layers) { rc = linear_add_norm(*L.w_down, c.hidden, c.inter, *pf_.gated, *pf_.r1, *pf_.x, *layers_[li + 1].rms_attn, *pf_.xn); }
        else if (rc == 0)
        {
            rc = linear(*L.w_down, c.hidden, c.inter, *pf_.gated, *pf_.o);
            if (rc == 0) { rc = hip_add_bf16(pf_.r1->data(), pf_.o->data(), pf_.x->data(), (unsigned long long)n * c.hidden); }
        }
    }
    if (rc != 0 || !last) { return rc; }
    // the head runs on the last token's state: its greedy pick becomes the current token at position pos0 + n
    // (the row copy rides on the launch stream behind the last layer)
    const int state[2] = { tokens[n - 1], pos0 + n - 1 };
    if (hipMemcpyAsync(x_->data(), (const char*)pf_.x->data() + (size_t)(n - 1) * c.hidden * 2, (size_t)c.hidden * 2, hipMemcpyDeviceToDevice, stream) != hipSuccess) { return 1; }
    if (GpuControl::copyHostToDevice(d_state_, state, sizeof(state)) != 0) { return 1; }
    return head();
}

double DecodeModel::run(int n_steps, int use_graph)
{
    if (n_steps <= 0 || currentPos() < 0 || currentPos() + n_steps > cfg_.t_kv) { return -2.0; }    // would run past the KV cache
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) { return -1.0; }
    double result = -1.0;
    const int sync_before = hip_quant_set_sync(0);
    if (use_graph)
    {
        hipStream_t stream = nullptr;
        hipGraph_t graph = nullptr;
        hipGraphExec_t exec = nullptr;
        if (hipStreamCreate(&stream) != hipSuccess)
        {
            hip_quant_set_sync(sync_before);
            return -4.0;
        }
        (void)hipDeviceSynchronize();
        hip_quant_set_stream(stream);
        bool ok = hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal) == hipSuccess;
        if (ok) { ok = step() == 0; }
        ok = (hipStreamEndCapture(stream, &graph) == hipSuccess) && ok;
        hip_quant_set_stream(nullptr);
        if (ok) { ok = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0) == hipSuccess; }
        if (ok)
        {
            (void)hipEventRecord(e0, stream);
            for (int s = 0; s < n_steps; s++) { ok = (hipGraphLaunch(exec, stream) == hipSuccess) && ok; }
            (void)hipEventRecord(e1, stream);
            ok = (hipEventSynchronize(e1) == hipSuccess) && ok;
        }
        if (ok)
        {
            float ms = 0;
            (void)hipEventElapsedTime(&ms, e0, e1);
            result = ms;
        }
        if (exec) { (void)hipGraphExecDestroy(exec); }
        if (graph) { (void)hipGraphDestroy(graph); }
        (void)hipStreamDestroy(stream);
    }
    else
    {
        bool ok = true;
        (void)hipEventRecord(e0, nullptr);
        for (int s = 0; s < n_steps; s++) { ok = (step() == 0) && ok; }
        (void)hipEventRecord(e1, nullptr);
        ok = (hipEventSynchronize(e1) == hipSuccess) && ok;
        if (ok)
        {
            float ms = 0;
            (void)hipEventElapsedTime(&ms, e0, e1);
            result = ms;
        }
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    hip_quant_set_sync(sync_before);
    return result;
}

}    // namespace cccc
