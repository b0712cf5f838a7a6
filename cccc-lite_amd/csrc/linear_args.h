// One quantized linear, normalised from the BLAS-style call of the unified dispatcher
// (cccc/cublas_real.h:875-880): y[t][o] = alpha * sum_k dequant(W)[o][k] * x[t][k] + beta * y[t][o].
#pragma once
#include <stdint.h>

namespace ccq
{

struct LinearArgs
{
    const uint8_t* W;         // quantized weight, row o starts at element o * ldw (FP4: two elements per byte)
    const uint8_t* blk_sc;    // FP4 per-block E4M3 scales over the flat element index, or nullptr
    const uint16_t* X;        // bf16 activations, token t starts at element t * ldx
    uint16_t* Y;              // bf16 output, element (t, o) at t * y_stride_tok + o * y_stride_out
    long long ldw;
    long long ldx;
    long long y_stride_tok;
    long long y_stride_out;
    int n_out;
    int tokens;
    int K;
    unsigned block_size;      // FP4 block length (elements)
    float w_scale;            // per-tensor dequant multiplier (invScale); ignored when blk_sc is set
    float alpha;
    float beta;
    // gate / up pair (gemm_mfma_direct_kernel<..., PAIR>): W is the gate weight, W_pair the up weight of the same shape
    // and layout; the output is the SwiGLU product of the two linears
    const uint8_t* W_pair;
    float w_scale_pair;
    // up to three linears of one K, type and layout on the same activations as one launch (gemm_mfma_direct_kernel<..., SEG>):
    // segment s owns the feature tiles seg_tile0[s] .. seg_tile0[s + 1] - 1 of the grid and brings its own weight, output,
    // width and scale; n_segments = 0 everywhere else
    int n_segments;
    const uint8_t* seg_W[3];
    uint16_t* seg_Y[3];
    int seg_n_out[3];
    int seg_tile0[4];
    float seg_w_scale[3];
    long long seg_y_stride_tok[3];
};

// What follows a k-split GEMM when its combine launch also carries the residual add and the RMSNorm behind it
// (gemm_splitk_combine_add_norm_kernel): rows of n_out values, all dense.
struct AddNormArgs
{
    const uint16_t* res;      // residual rows [tokens][n_out]
    uint16_t* sum;            // bf16(res + bf16(W x))
    const uint16_t* norm_w;   // [n_out]
    uint16_t* y;              // rmsnorm(sum) * norm_w
    float eps;
};

}    // namespace ccq
