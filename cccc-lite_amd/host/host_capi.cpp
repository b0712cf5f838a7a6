// Plain-C window onto the host mirror so that tests and the benchmark (Python, ctypes) drive the
// same Matrix::mulBatched path a cccc graph would.
#include "DecodeModel.h"
#include <cstring>
#include "Matrix.h"
#include "../../include/cccc_hip_quant.h"
#include <hip/hip_runtime.h>
#include <cstdio>
#include <vector>

using namespace cccc;

extern "C" {

int cccc_host_init(int device) { return GpuControl::select(device) ? 0 : 1; }

void* cccc_matrix_create(int w, int h, int c, int n, int dtype)
{
    if (!GpuControl::getCurrentGpu()) { GpuControl::select(0); }
    return new Matrix(w, h, c, n, (DataType)dtype);
}

void cccc_matrix_destroy(void* m) { delete (Matrix*)m; }

void* cccc_matrix_data(void* m) { return ((Matrix*)m)->data(); }

int cccc_matrix_upload(void* m, const void* host, size_t bytes) { return ((Matrix*)m)->copyFromHost(host, bytes); }

int cccc_matrix_download(void* m, void* host, size_t bytes) { return ((Matrix*)m)->copyToHost(host, bytes); }

int cccc_matrix_load_quantized(void* m, const void* host, long long n_bytes, float scale, int dtype)
{
    ((Matrix*)m)->loadQuantizedDirect((const uint8_t*)host, n_bytes, scale, (DataType)dtype);
    return 0;
}

int cccc_matrix_set_block_scale(void* m, const void* host, long long n_scales)
{
    ((Matrix*)m)->setBlockScaleFromHost(host, n_scales);
    return ((Matrix*)m)->getBlockScaleData() ? 0 : 1;
}

int cccc_matrix_quantize(void* m, int dtype)
{
    ((Matrix*)m)->quantizeWeights((DataType)dtype);
    return 0;
}

// 0 / 1: build tiled copies of FP8 linear weights when they are loaded or quantized (default 1)
void cccc_host_set_repack(int enabled) { MatrixData::repack_weights = enabled != 0; }

// (re)builds the tiled copy of an FP8 weight matrix whose bytes were written straight into its storage
int cccc_matrix_prepare_tiled(void* m)
{
    Matrix* mat = (Matrix*)m;
    mat->prepareTiled();
    return mat->hasTiled() ? 0 : 1;
}

int cccc_matrix_dtype(void* m) { return (int)((Matrix*)m)->getDataType(); }

float cccc_matrix_quant_scale(void* m) { return ((Matrix*)m)->getQuantScale(); }

void cccc_matrix_set_quant_scale(void* m, float scale) { ((Matrix*)m)->setQuantScale(scale); }

const void* cccc_matrix_block_scale_data(void* m) { return ((Matrix*)m)->getBlockScaleData(); }

long long cccc_matrix_get_block_scale(void* m, void* host, long long capacity)
{
    Matrix* mat = (Matrix*)m;
    if (!mat->getBlockScaleData()) { return 0; }
    const long long count = mat->getBlockScaleCount();
    if (count > capacity) { return -count; }
    mat->getBlockScaleToHost(host);
    return count;
}

int cccc_matrix_mul(void* A, void* B, void* R, float a, float r, int ta, int tb)
{
    return Matrix::mul(*(Matrix*)A, *(Matrix*)B, *(Matrix*)R, a, r, (MatrixTransType)ta, (MatrixTransType)tb);
}

int cccc_matrix_mul_batched(void* A, void* B, void* R, int ta, int tb, float a, float r)
{
    return Matrix::mulBatched(*(Matrix*)A, *(Matrix*)B, *(Matrix*)R, (MatrixTransType)ta, (MatrixTransType)tb, a, r);
}

unsigned long long cccc_gpu_allocated_bytes(void)
{
    GpuControl* g = GpuControl::getCurrentGpu();
    return g ? (unsigned long long)g->allocatedBytes() : 0ull;
}

// ---- weight container

void* cccc_weightfile_open(const char* path, int* status)
{
    auto* f = new WeightFile();
    const int rc = f->parseFile(path);
    if (status) { *status = rc; }
    if (rc != 0)
    {
        delete f;
        return nullptr;
    }
    return f;
}

void cccc_weightfile_close(void* f) { delete (WeightFile*)f; }

int cccc_weightfile_count(void* f) { return (int)((WeightFile*)f)->keys().size(); }

const char* cccc_weightfile_key(void* f, int i)
{
    const auto& keys = ((WeightFile*)f)->keys();
    return (i >= 0 && i < (int)keys.size()) ? keys[i].c_str() : nullptr;
}

// Copies up to `capacity` bytes of the entry to dst (dst may be NULL); returns its length, -1 when absent.
long long cccc_weightfile_get(void* f, const char* key, void* dst, unsigned long long capacity)
{
    auto [p, n] = ((WeightFile*)f)->get_value(key);
    if (!p && !((WeightFile*)f)->has_value(key)) { return -1; }
    if (dst && n) { std::memcpy(dst, p, n < capacity ? n : (size_t)capacity); }
    return (long long)n;
}

// Resolves a weight name: writes the key into key_out (NUL-terminated, truncated to capacity) and returns the
// dtype, with bit 16 set when the entry is quantized; -1 when the name is not in the file.
int cccc_weightfile_resolve(void* f, const char* name, char* key_out, int capacity)
{
    const auto wk = ((WeightFile*)f)->resolve(name);
    if (!wk.valid()) { return -1; }
    if (key_out && capacity > 0)
    {
        std::strncpy(key_out, wk.key.c_str(), (size_t)capacity - 1);
        key_out[capacity - 1] = 0;
    }
    return (int)wk.dt | (wk.is_quant ? 0x10000 : 0);
}

// names: NUL-separated list ending with an empty string
int cccc_weightfile_load_named_group(void* f, void* m, const char* names)
{
    std::vector<std::string> list;
    for (const char* p = names; p && *p; p += std::strlen(p) + 1) { list.emplace_back(p); }
    return ((WeightFile*)f)->loadNamedGroup(*(Matrix*)m, list);
}

// A new Matrix handle viewing rows [row0, row0 + n_rows) of m (NULL when the range does not fit); destroy it like any other.
void* cccc_matrix_rows_view(void* m, int row0, int n_rows)
{
    Matrix v = ((Matrix*)m)->rowsView(row0, n_rows);
    return v.data() ? new Matrix(v) : nullptr;
}

int cccc_weightfile_load_named(void* f, void* m, const char* name) { return ((WeightFile*)f)->loadNamed(*(Matrix*)m, name); }

unsigned char cccc_host_float_to_e4m3(float v) { return floatToE4m3Truncated(v); }

unsigned short cccc_host_half_to_bf16(unsigned short h) { return halfBitsToBf16Truncated(h); }

// ---- decode model

void* cccc_decode_create(int layers, int hidden, int n_q, int n_kv, int head_dim, int inter, int vocab, int t_kv, float theta, float eps)
{
    if (!GpuControl::getCurrentGpu()) { GpuControl::select(0); }
    if (head_dim != 128 || hidden % 16 != 0 || inter % 16 != 0 || n_kv <= 0 || n_q % n_kv != 0) { return nullptr; }
    const DecodeConfig cfg{ layers, hidden, n_q, n_kv, head_dim, inter, vocab, t_kv, theta, eps };
    return new DecodeModel(cfg, GpuControl::getCurrentGpu());
}

void cccc_decode_destroy(void* m) { delete (DecodeModel*)m; }

int cccc_decode_set_tensor(void* m, int layer, int which, const void* host, unsigned long long bytes, int dtype, float scale)
{
    return ((DecodeModel*)m)->setTensor(layer, which, host, (size_t)bytes, (DataType)dtype, scale);
}

int cccc_decode_set_block_scales(void* m, int layer, int which, const void* host, unsigned long long n_scales)
{
    return ((DecodeModel*)m)->setBlockScales(layer, which, host, (size_t)n_scales);
}

void* cccc_decode_tensor_data(void* m, int layer, int which)
{
    Matrix* t = ((DecodeModel*)m)->tensor(layer, which);
    return t ? t->data() : nullptr;
}

int cccc_decode_quantize_linear(void* m, int layer, int which, const void* device_bf16, int to)
{
    return ((DecodeModel*)m)->quantizeLinear(layer, which, device_bf16, (DataType)to);
}

float cccc_decode_tensor_scale(void* m, int layer, int which)
{
    Matrix* t = ((DecodeModel*)m)->tensor(layer, which);
    return t ? t->getQuantScale() : 0.0f;
}

int cccc_decode_tensor_prepare(void* m, int layer, int which)
{
    Matrix* t = ((DecodeModel*)m)->tensor(layer, which);
    if (!t) { return -1; }
    t->prepareTiled();
    return t->hasTiled() ? 0 : 1;
}

int cccc_decode_load_named(void* m, void* f, int quantize_to, char* failed_out, int capacity)
{
    std::string failed;
    const int rc = ((DecodeModel*)m)->loadNamedWeights(*(WeightFile*)f, (DataType)quantize_to, &failed);
    if (failed_out && capacity > 0)
    {
        std::strncpy(failed_out, failed.c_str(), (size_t)capacity - 1);
        failed_out[capacity - 1] = 0;
    }
    return rc;
}

int cccc_decode_save_named(void* m, const char* path) { return ((DecodeModel*)m)->saveNamedWeights(path); }

// Writes one matrix as a named weight (with its scale / block scales) into a container of its own.
int cccc_matrix_save_named(void* m, const char* name, const char* path)
{
    WeightFileWriter w;
    w.set_value("named_weights", std::string("1"));
    addNamedWeight(w, name, *(Matrix*)m);
    return w.save(path) > 0 ? 0 : -1;
}

void cccc_decode_set_exact_attention(void* m, int exact) { ((DecodeModel*)m)->setExactAttention(exact != 0); }
void cccc_decode_set_qk_norm(void* m, int on) { ((DecodeModel*)m)->setQkNorm(on != 0); }
int cccc_decode_qk_norm(void* m) { return ((DecodeModel*)m)->qkNorm() ? 1 : 0; }
void cccc_decode_set_repack_linears(void* m, int on) { ((DecodeModel*)m)->setRepackLinears(on != 0); }
void cccc_decode_set_tied_lm_head(void* m, int tied) { ((DecodeModel*)m)->setTiedLmHead(tied != 0); }
int cccc_decode_tied_lm_head(void* m) { return ((DecodeModel*)m)->tiedLmHead() ? 1 : 0; }

int cccc_decode_prefill(void* m, const int* tokens, int n_tokens, int pos0) { return ((DecodeModel*)m)->prefill(tokens, n_tokens, pos0); }

int cccc_decode_reset(void* m, int token, int pos) { return ((DecodeModel*)m)->reset(token, pos); }

int cccc_decode_step(void* m)
{
    const int rc = ((DecodeModel*)m)->step();
    return (hipDeviceSynchronize() == hipSuccess) ? rc : 1;
}

double cccc_decode_run(void* m, int n_steps, int use_graph) { return ((DecodeModel*)m)->run(n_steps, use_graph); }

int cccc_decode_token(void* m) { return ((DecodeModel*)m)->currentToken(); }

int cccc_decode_pos(void* m) { return ((DecodeModel*)m)->currentPos(); }

int cccc_decode_logits(void* m, void* host, unsigned long long bytes) { return ((DecodeModel*)m)->logits().copyToHost(host, (size_t)bytes); }

int cccc_decode_activation(void* m, int which, void* host, unsigned long long bytes)
{
    Matrix* a = ((DecodeModel*)m)->activation(which);
    return a ? a->copyToHost(host, (size_t)bytes) : -1;
}

int cccc_decode_kv(void* m, int layer, int is_v, void* host, unsigned long long bytes)
{
    DecodeModel* d = (DecodeModel*)m;
    return (is_v ? d->vCache(layer) : d->kCache(layer)).copyToHost(host, (size_t)bytes);
}

void* cccc_decode_kv_data(void* m, int layer, int is_v)
{
    DecodeModel* d = (DecodeModel*)m;
    if (layer < 0 || layer >= d->config().layers) { return nullptr; }
    return (is_v ? d->vCache(layer) : d->kCache(layer)).data();
}

int cccc_decode_cos_table(void* m, void* host, unsigned long long bytes) { return ((DecodeModel*)m)->cosTable().copyToHost(host, (size_t)bytes); }

unsigned long long cccc_decode_weight_bytes(void* m) { return (unsigned long long)((DecodeModel*)m)->weightBytes(); }

}    // extern "C"
