// Batch-1 decode step of a Qwen3-style transformer with weight-only quantized linears, driven from
// the host mirror: what the reference does per token through MainProcess::testExternalData ->
// Net::inference -> MatrixOp::forward (cccc/MainProcess.cpp:1171-1239, cccc/Net.cpp:1748-1792,
// cccc/MatrixOp.cpp:12-26) for the graph of scripts/convert_weights.py:488-692, collapsed into
// six launches per layer and two per token (lm_head with the greedy candidates; pick + next embedding).  Token id and position live in device memory, so a step is a fixed
// launch sequence that can be replayed as one hipGraph.
#pragma once
#include "Matrix.h"
#include "WeightFile.h"
#include <string>
#include <memory>
#include <vector>

namespace cccc
{

struct DecodeConfig
{
    int layers, hidden, n_q, n_kv, head_dim, inter, vocab, t_kv;
    float theta, eps;
};

class DecodeModel
{
public:
    enum Tensor
    {
        RMS_ATTN = 0, WQ, WK, WV, Q_NORM, K_NORM, WO, RMS_FFN, W_GATE, W_UP, W_DOWN,    // per layer
        EMB = 100, RMS_FINAL, LM_HEAD                                                    // global (layer ignored)
    };

    DecodeModel(const DecodeConfig& cfg, GpuControl* gpu);
    ~DecodeModel();

    // Intermediate BF16 vectors of the step in flight (what the last layer that ran left in them)
    enum Activation
    {
        ACT_X = 0, ACT_R1, ACT_Q, ACT_K, ACT_V, ACT_ATT, ACT_GATED
    };

    const DecodeConfig& config() const { return cfg_; }
    Matrix* tensor(int layer, int which);
    Matrix* activation(int which);

    // Uploads file bytes: FP8 codes or packed FP4 nibbles for the linears (loadQuantizedDirect), BF16 bits for norms / embedding.
    int setTensor(int layer, int which, const void* host, size_t bytes, DataType dt, float scale);
    // FP4 linears: the E4M3 block scales that go with the packed codes (one byte per 16 elements).
    int setBlockScales(int layer, int which, const void* host, size_t n_scales);

    // Quantizes one linear on the device from BF16 values already there ([n_out][K], the tensor's shape): the reference's
    // on-the-fly route for a model stored unquantized (Net::quantizeWeights -> Matrix::quantizeWeights,
    // cccc/Net.cpp:1142-1233, cccc/Matrix.cpp:301-355) -- FP8 with the per-tensor scale absmax / max_code and truncating
    // encoders, FP4 with per-block E4M3 scales.  0 ok, -1 not a linear of this model / not a quantized type, -3 the
    // tensor is too small to quantize (a side under 64).
    int quantizeLinear(int layer, int which, const void* device_bf16, DataType to);

    // Loads every tensor from a converted model file by the converter's names (scripts/convert_weights.py:142-166):
    // W_emb, W_rms_final, W_lm_head (absent: tied embeddings, the head then reads W_emb in BF16), W_rms_attn_<i>, W_q_<i>, W_k_<i>, W_v_<i>, W_o_<i>,
    // W_qnorm_<i>, W_knorm_<i> (a file without them loads as a model without per-head norms), W_rms_ffn_<i>, W_gate_<i>,
    // W_up_<i>, W_down_<i>.  FP8 and FP4 linears are taken as stored;
    // linears stored as BF16 / HALF / FLOAT are quantized on load to `quantize_to` with a per-tensor absmax scale
    // (the reference's weight_data_type route, cccc/Matrix.cpp:301-355).  0 ok; otherwise `failed` names the tensor:
    // -1 missing, -2 wrong size, -3 something the fused decode kernels do not take (FP4 without block scales, a tensor too
    // small to quantize).  Every tensor keeps the format the file gives it (cccc/Net.cpp:1444-1481 resolves each by
    // itself): projections that share a launch but not a format (q, k, v; gate, up) go out as separate launches.  FP4_E2M1 linears load with their blockscale_<name> entries.
    int loadNamedWeights(const WeightFile& file, DataType quantize_to = FP8_E5M2, std::string* failed = nullptr);

    // Writes every tensor under the same names, as Net::saveNamedWeights does (cccc/Net.cpp:1235-1314): the header
    // entry "data_type" (the linears' type), then per tensor "weight_<dtype>_<name>" with its bytes as they sit on the
    // device, "scale_<name>" when the per-tensor scale is not 1 and "blockscale_<name>" for FP4.  This is the cache the
    // reference writes after quantizing on load (save_fp8_file, cccc/MainProcess.cpp:362-378): loading it back gives
    // the same bytes without quantizing again.  0 ok, -1 the file could not be written.
    int saveNamedWeights(const std::string& filename);

    // false (default): two-launch attention with the norm / RoPE / append folded in and FP32 probabilities;
    // true: the reference's rounding points throughout (BF16 probabilities over the whole row; three launches).
    void setExactAttention(bool exact) { exact_attention_ = exact; }
    // Per-head RMSNorm of q and k in front of the rotation: on for Qwen3-style models (default), off for models without
    // W_qnorm / W_knorm such as Llama-3.1 (has_qknorm in scripts/convert_weights.py:488-530).  loadNamedWeights sets it
    // from what the file holds.
    void setQkNorm(bool on) { qk_norm_ = on; }
    // Tied embeddings (tie_word_embeddings, scripts/convert_weights.py:230-260: no W_lm_head entry in the file): the head
    // multiplies by the BF16 embedding table itself, as the reference does -- it never quantizes an EMBED table nor a view
    // sharing its storage (cccc/Net.cpp:1158-1190) -- and no separate head is stored.  loadNamedWeights sets it from the file.
    void setTiedLmHead(bool tied);
    // Keep the load-time tiled copy of every linear, not only of the head: the decode step does not read them (its per-layer
    // kernels stay on the file layout), the prompt phase's GEMMs run 1.10-1.15x faster on them (FP4: the register-fed GEMM
    // needs them at all), and the weights take twice the memory.  Off by default; takes effect for tensors set or loaded
    // afterwards.
    void setRepackLinears(bool on) { repack_linears_ = on; }
    bool tiedLmHead() const { return tied_lm_head_; }
    bool qkNorm() const { return qk_norm_; }
    int reset(int token, int pos);          // sets the device-side token / position and fetches the token's embedding (KV caches are kept)
    int step();                             // enqueues one decode step; the next token replaces the current one
    // The prompt phase: n tokens at positions pos0 .. pos0 + n - 1 in one pass per layer -- what the reference's graph does
    // when cccc-llm feeds it the whole prompt (cccc-llm/cccc-llm.cpp:589-618): the linears through Rocblas::gemm with n
    // columns (the matrix-core GEMM from 48 tokens on), the per-head norm / RoPE / cache append, the causal attention with
    // the reference's rounding points, residual adds and the SwiGLU product as row kernels.  Afterwards the caches hold
    // the prompt, the current token is the greedy pick after its last token and the position is pos0 + n: step() carries
    // on from there.  Prompts longer than 2048 tokens go through in pieces of 2048.  0 ok, -1 bad arguments.
    int prefill(const int* tokens, int n_tokens, int pos0);
    // Runs n steps; use_graph: capture one step and replay it.  Returns elapsed ms (events on the launch stream) or < 0.
    double run(int n_steps, int use_graph);
    int currentToken();                     // blocking 4-byte read
    int currentPos();
    Matrix& logits() { return *logits_; }
    Matrix& kCache(int layer) { return *k_cache_[layer]; }
    Matrix& vCache(int layer) { return *v_cache_[layer]; }
    Matrix& cosTable() { return *cos_; }
    size_t weightBytes() const;

private:
    struct Layer
    {
        std::unique_ptr<Matrix> rms_attn, wq, wk, wv, q_norm, k_norm, wo, rms_ffn, w_gate, w_up, w_down;
    };
    DecodeConfig cfg_;
    GpuControl* gpu_;
    std::vector<Layer> layers_;
    std::unique_ptr<Matrix> emb_, rms_final_, lm_head_, logits_, cos_, sin_;
    std::vector<std::unique_ptr<Matrix>> k_cache_, v_cache_;
    std::unique_ptr<Matrix> x_, r1_, q_, k_, v_, att_, gated_, attn_ws_, argmax_ws_;
    std::unique_ptr<Matrix> gate_, up_;     // only for a layer whose gate and up weights differ in format (allocated on first use)
    // activations of a prompt piece, grown on demand: [tokens][features] BF16, and the token ids as floats (hip_embed_fwd's input)
    struct PromptBuffers
    {
        int tokens = 0;
        std::unique_ptr<Matrix> ids, x, xn, q, k, v, q_rot, att, o, r1, gate, up, gated;
    } pf_;
    int prefillPiece(const int* tokens, int n, int pos0, bool last);
    int head();                             // final norm + lm_head + greedy pick + next embedding on x_
    unsigned long long attn_ws_bytes_ = 0;
    bool exact_attention_ = false;
    bool qk_norm_ = true;
    bool tied_lm_head_ = false;
    bool repack_linears_ = false;
    int* d_state_ = nullptr;    // [0] token, [1] position
};

}    // namespace cccc
