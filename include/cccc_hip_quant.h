/*
 * cccc_hip_quant.h -- C-ABI of the MI355X (gfx950) weight-only quantized linear path for cccc.
 *
 * Conventions are those of the reference's HIP kernel library (cccc-hip/hip_functions.h:3-9,
 * cccc-hip/hip_functions.cpp:32-42):
 *   - plain C linkage, plain pointers and sizes, `int` return:
 *        0  success
 *        1  HIP runtime / launch error (a message is written to stderr)
 *       -1  unsupported type pair or argument combination (nothing was launched)
 *   - data types are passed as `int` holding a cccc::DataType value (cccc/types.h:24-34):
 *        0 float, 1 double, 2 half, 3 bfloat16, 4 fp8_e4m3, 5 fp8_e5m2, 6 fp4_e2m1
 *   - all pointers are device pointers owned by the caller; the library never frees them.
 *   - work is enqueued on the library stream (the null stream unless hip_quant_set_stream was
 *     called).  The reference synchronises the device after every kernel; here that is a switch
 *     (hip_quant_set_sync), off by default, because stream order on one stream is observationally
 *     the same for a caller that reads results with blocking copies (cccc/MatrixData.cpp:155-165).
 */
#pragma once

#ifndef C_EXPORT
#ifdef __cplusplus
#define C_EXPORT extern "C"
#else
#define C_EXPORT
#endif
#endif

/* cccc::DataType values (cccc/types.h:24-34) */
#define CCCC_FLOAT    0
#define CCCC_DOUBLE   1
#define CCCC_HALF     2
#define CCCC_BFLOAT16 3
#define CCCC_FP8_E4M3 4
#define CCCC_FP8_E5M2 5
#define CCCC_FP4_E2M1 6

/* MatrixTransType values (cccc/blas_types.h): 0 = no-trans, 1 = trans */
#define CCCC_NO_TRANS 0
#define CCCC_TRANS    1

/*
 * Unified type conversion, `n` elements, result multiplied by `scale` where the pair is a
 * (de)quantisation.  Replaces the float/half/bf16-only hip_convert of the reference
 * (cccc-hip/hip_functions.h:179-181, cccc-hip/hip_functions.cpp:2681-2690) with the full table of
 * cuda_convert (cccc-cuda/cuda_functions.h:218-224, cccc-cuda/cuda_functions.cu:3066-3090):
 *   float -> bf16 | e4m3 | e5m2 | fp4        half -> float | bf16       bf16 -> float | half | e4m3
 *   e4m3 | e5m2 -> float | half | bf16       fp4 -> float | bf16
 * Same type with scale == 1 copies `n` BYTES, as the reference does.  FP4 buffers hold two
 * elements per byte, low nibble = even element (cccc/types.h:257-261).
 */
C_EXPORT int hip_convert(const void* src, int src_type, void* dst, int dst_type, unsigned int n, float scale);

/*
 * Packed FP4_E2M1 nibbles + one FP8_E4M3 scale byte per `block_size` consecutive (flat) elements
 * -> BF16.  HIP twin of cuda_fp4_blockscale_to_bf16 (cccc-cuda/cuda_functions.h:232-233,
 * cccc-cuda/cuda_functions.cu:2926-2939, :2953-2960).
 */
C_EXPORT int hip_fp4_blockscale_to_bf16(const void* src_nibbles, const void* src_scales, void* dst,
                                        unsigned int n_elems, unsigned int block_size);

/*
 * float -> packed FP4_E2M1 nibbles + FP8_E4M3 (truncating) dequant scale per block.  HIP twin of
 * cuda_float_to_fp4_blockscale (cccc-cuda/cuda_functions.h:230-231,
 * cccc-cuda/cuda_functions.cu:2896-2923, :2943-2950).
 */
C_EXPORT int hip_float_to_fp4_blockscale(const void* src, void* dst_nibbles, void* dst_scales,
                                         unsigned int n_elems, unsigned int block_size);

/*
 * Largest |x| of `n` elements (float, half or bf16) written as one float to device memory at
 * `d_result`.  Stands in for the cuBLAS iamax + 4-byte copy that Matrix::quantizeWeights uses to
 * derive the per-tensor FP8 scale (cccc/Matrix.cpp:338-343).  NaNs are ignored.
 */
C_EXPORT int hip_absmax(const void* src, int src_type, unsigned int n, void* d_result);

/*
 * Unified quantized GEMM, column-major:  C[M x N] = alpha * op(A)[M x K] * op(B)[K x N] + beta * C.
 * Carries the arguments of the reference's unified dispatcher Cublas::gemm
 * (cccc/cublas_real.h:875-880) plus the FP4 block size that the reference hard-codes as 16
 * (cccc/cublas_real.h:953, :1076).  It is what Matrix::mul / Matrix::mulBatched hand to
 * `gpu()->cublas_->gemm(...)` (cccc/Matrix.cpp:1130-1133, :1199-1202); a HIP build calls it from
 * Rocblas::gemm.  Implemented branches: exactly one of A / B quantized (types 4, 5, 6), the other
 * BF16, C BF16 -- the W8A16 / FP4 branches cccc/cublas_real.h:943-964 (weight is A) and
 * :1066-1087 (weight is B).  Semantics are the reference's: the weight is dequantised to BF16
 * (times invScale, or times its per-block E4M3 scale when blk_sc is given for FP4), multiplied
 * with FP32 accumulation, alpha/beta applied in FP32, rounded once to BF16.  The HALF twin of the
 * FP8 branches is implemented as well (cccc/cublas_real.h:921-938: FP8 weight, the other operand and
 * C of type HALF; the weight is dequantised to half, FP32 accumulation, one rounding to half).
 * `act_scale` is accepted and ignored (it only drives the W8A8 route, cccc/cublas_real.h:871-873).
 * Anything else (both operands quantized, FP4 with HALF, mixed 16-bit types, other C types) returns -1.
 * Device memory: the one case in which the library allocates is a GEMM of 17 tokens or more (FP8, FP4 on a tiled
 * copy, or HALF activations) whose output has too few tiles to fill the GPU; it then splits K over workgroups and keeps
 * FP32 partial sums in a scratch buffer per (host thread, device, stream) that grows on demand and lives until the
 * process ends (at most 16 * M * N * 4 bytes).  While the stream is being captured into a graph the buffer is never
 * grown: the call then runs without the split (see hip_quant_workspace_reserve).
 */
C_EXPORT int hip_quant_gemm(int transA, int transB, int M, int N, int K, float alpha,
                            const void* A, int typeA, int lda, float invScaleA,
                            const void* B, int typeB, int ldb, float invScaleB,
                            float beta, void* C, int typeC, int ldc, float act_scale,
                            const void* blk_scA, const void* blk_scB, unsigned int block_size);

/*
 * hip_quant_gemm for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments,
 * kernels and results as hip_quant_gemm; the only difference is where the k-split GEMM keeps its FP32
 * partial sums: in a static device array of HIP_QUANT_NOALLOC_SCRATCH_BYTES inside the library (one per
 * GPU the library runs on, held until the process ends) instead of a buffer grown on demand.  The call
 * never allocates or frees device memory.  A shape whose k-split needs more than that (splits * M * N * 4
 * bytes, splits <= 16) returns -1 with a message on stderr and launches nothing; 32 MiB covers 512 tokens x 4096
 * features.  The routes that split K, all with few output tiles for the GPU: FP8 GEMMs of 17 tokens or more (K % 64 == 0),
 * FP4 GEMMs of 17 tokens or more on a registered tiled copy (K % 128 == 0), and HALF-activation GEMMs of 17 tokens or more.
 * Every call on a GPU shares the one array: calls that overlap on one GPU (two streams, two host
 * threads) race on it and must be ordered by the caller.  Nothing in it needs clearing between calls:
 * each call overwrites every partial sum it later reads.
 */
#define HIP_QUANT_NOALLOC_SCRATCH_BYTES (32u << 20)
C_EXPORT int hip_quant_gemm_noalloc(int transA, int transB, int M, int N, int K, float alpha,
                                    const void* A, int typeA, int lda, float invScaleA,
                                    const void* B, int typeB, int ldb, float invScaleB,
                                    float beta, void* C, int typeC, int ldc, float act_scale,
                                    const void* blk_scA, const void* blk_scB, unsigned int block_size);

/*
 * Optional load-time repack (no counterpart in the reference; the on-disk format and the caller's
 * weight buffer are left untouched).  hip_quant_weight_prepare writes an MI355X-friendly tiled copy
 * of an FP8 weight W ([n_out][ldw], K contiguous, as loadQuantizedDirect uploads it) into `dst_tiled`
 * -- caller-owned device memory of hip_quant_tiled_size(...) bytes -- and remembers it under the key
 * `W`.  Later hip_quant_gemm calls whose weight pointer, type and shape match may use the tiled copy
 * (today: up to 16 tokens, except one or two tokens on weights under 8 MiB, and the GEMM of 17 tokens or
 * more when K is a multiple of 64): the matrix-core kernels want the 16 rows x 64 codes of one load
 * instruction to be one contiguous KiB.
 * Results agree with the row-major kernels up to the FP32 summation order.  The copy is keyed on the pointer, not
 * on the bytes behind it: after any write to W the caller must call hip_quant_weight_prepare again (or
 * hip_quant_weight_release), otherwise later calls compute from the stale copy.  hip_quant_weight_release forgets
 * the key (before the caller frees either buffer).  Returns 0 ok, 1 runtime error, -1 unsupported (K % 16 != 0, ...;
 * FP4 weights have an entry point of their own below).
 */
C_EXPORT unsigned long long hip_quant_tiled_size(int type, int n_out, int K);
C_EXPORT int hip_quant_weight_prepare(const void* W, int type, int n_out, int K, int ldw, void* dst_tiled);
C_EXPORT int hip_quant_weight_release(const void* W);
/* The same for an FP4_E2M1 weight W ([n_out][K / 2] packed codes, K % 32 == 0) with its E4M3 block scales
 * (one byte per block_size = 16 or 32 elements of the flat index): the tiled copy holds codes and scales
 * (hip_quant_tiled_size(6, n_out, K) bytes) in the order the matrix-core GEMV for 1..16 tokens consumes
 * them.  hip_quant_gemm uses it when the weight pointer, the block-scale pointer, the block size and the
 * shape match.  Same rule: prepare again after any write to the codes or the scales. */
C_EXPORT int hip_quant_weight_prepare_fp4(const void* W, const void* blk_sc, unsigned int block_size, int n_out, int K, void* dst_tiled);

/* ------------------------------------------------------------------------------------------------
 * Decode-step neighbours of the linear (BF16 activations, one new token).
 *
 * hip_rms_norm_fwd, hip_rope_fwd and hip_embed_fwd keep the reference's signatures
 * (cccc-hip/hip_functions.h:79-80, :91-94, :112-113) and semantics for type 3 (BF16); other types
 * return 1 with a message, as the reference does for unsupported types.  hip_embed_fwd reads float ids.
 */
C_EXPORT int hip_rms_norm_fwd(int type, void* X, void* Y, void* scale, void* invstd_out,
                              unsigned int outer, unsigned int inner, float epsilon);
C_EXPORT int hip_rope_fwd(int type, const void* X, void* Y, const void* cos_tab, const void* sin_tab,
                          unsigned int D, unsigned int T, unsigned int B, unsigned int pos_offset);
C_EXPORT int hip_embed_fwd(int type, const void* ids, const void* W, void* Y, int D, int T, int B);

/*
 * Fused pieces of a Qwen3-style decode step (no single counterpart in the reference, which runs the
 * graph op by op: scripts/convert_weights.py:488-692, cccc/MatrixOp.cpp:104-280).  Each keeps the
 * rounding points of the ops it replaces: every intermediate the reference stores as a BF16 tensor
 * is rounded to BF16 here too.  The step position and the current token id live in device memory
 * (`d_pos`, `d_token`: one int32 each) so that a step is a fixed launch sequence.
 */

/* y_s = W_s * [rmsnorm](x) for 1..3 quantized weights sharing x (q/k/v), or the SwiGLU pair
 * y = bf16(silu(W[0] x) * (W[1] x)) with silu(g) = bf16(g * bf16(sigmoid g)); optional residual
 * y = bf16(y + residual) on W[0]'s output.  Weights are [n_out][K], K contiguous, K % 16 == 0; FP4_E2M1
 * weights (two elements per byte, K % 32 == 0) come with their E4M3 block scales, one byte per block_size
 * (16 or 32) elements of the flat index, as cuda_fp4_blockscale_to_bf16 reads them
 * (cccc-cuda/cuda_functions.cu:2926-2939); w_scale is ignored for them. */
typedef struct hip_fused_linear
{
    int w_type;              /* 4 (FP8_E4M3), 5 (FP8_E5M2), 6 (FP4_E2M1 with block scales), or 3 (BF16: a weight the
                              * reference leaves unquantized -- a tied lm_head is the embedding table, cccc/Net.cpp:1158-1190;
                              * w_scale must be 1) */
    int K;
    int n_segments;          /* 1..3; 2 when pair != 0 */
    int pair;                /* 1: SwiGLU pair of W[0] (gate) and W[1] (up), both n_out[0] rows, into Y[0] */
    const void* W[3];
    int n_out[3];
    float w_scale[3];        /* per-tensor dequant multipliers (1.0f when absent) */
    void* Y[3];              /* bf16 [n_out[s]] */
    const void* X;           /* bf16 [K] */
    const void* norm_weight; /* bf16 [K] or NULL */
    float norm_eps;
    const void* residual;    /* bf16 [n_out[0]] or NULL */
    const void* blk_sc[3];   /* FP4 only: block scales of W[s] */
    unsigned int block_size; /* FP4 only: 16 or 32 */
    void* argmax_workspace;  /* single segment, no pair: the launch also leaves the greedy-pick candidates of its
                              * outputs here (hip_argmax_workspace_bytes(n_out[0]) bytes, 16-byte aligned) for
                              * hip_argmax_pick_embed_bf16; NULL: none */
} hip_fused_linear;
C_EXPORT int hip_quant_linear_fused(const hip_fused_linear* desc);

/* Per-head RMSNorm of q and k, RoPE at row *d_pos of the tables, append of k and v to the caches
 * (layout [kv_head][t_kv][128], the reference's (128, T_kv, 1, Hkv) cache).  head_dim is 128.
 * q_norm_w and k_norm_w both NULL: no per-head norm, the projections are rotated as they are (the
 * graph scripts/convert_weights.py:488-530 emits with has_qknorm = False, e.g. Llama-3.1). */
C_EXPORT int hip_qk_norm_rope_kv_bf16(const void* q, const void* k, const void* v,
                                      const void* q_norm_w, const void* k_norm_w,
                                      const void* cos_tab, const void* sin_tab,
                                      void* q_out, void* k_cache, void* v_cache,
                                      int n_q_heads, int n_kv_heads, int head_dim, int t_kv,
                                      const void* d_pos, float epsilon);

/* GQA attention of one query token over cache rows 0..*d_pos: scores rounded to BF16, FP32 softmax,
 * BF16 probabilities, y = bf16(V p).  Three launches over blocks of 64 cache rows; the caller owns the
 * workspace (16-byte aligned, hip_attention_decode_workspace_bytes(...) bytes; its content between
 * calls does not matter).  n_q_heads / n_kv_heads must be 1, 2 or 4; calls sharing one workspace
 * must be ordered on the stream. */
C_EXPORT unsigned long long hip_attention_decode_workspace_bytes(int n_q_heads, int n_kv_heads, int t_kv);
C_EXPORT int hip_attention_decode_bf16(const void* q, const void* k_cache, const void* v_cache, void* y,
                                       void* workspace, unsigned long long workspace_bytes,
                                       int n_q_heads, int n_kv_heads, int head_dim, int t_kv,
                                       const void* d_pos);

/* The q/k RMSNorm, RoPE, cache append and attention of one new token in two launches: q, k, v are the
 * raw projections ([n_q_heads][128], [n_kv_heads][128]); row *d_pos of both caches is written.  Same
 * workspace as above.  Scores are rounded to BF16 as in the reference; the softmax probabilities stay
 * FP32 (the reference rounds them to BF16 before the product with V), so outputs can differ from
 * hip_qk_norm_rope_kv_bf16 + hip_attention_decode_bf16 by about one BF16 ulp.  t_kv <= 65536.
 * q_norm_w and k_norm_w both NULL: no per-head norm, as above. */
C_EXPORT int hip_attention_decode_fused_bf16(const void* q, const void* k, const void* v,
                                             const void* q_norm_w, const void* k_norm_w,
                                             const void* cos_tab, const void* sin_tab,
                                             void* k_cache, void* v_cache, void* y,
                                             void* workspace, unsigned long long workspace_bytes,
                                             int n_q_heads, int n_kv_heads, int head_dim, int t_kv,
                                             const void* d_pos, float epsilon);

/* hip_qk_norm_rope_kv_bf16 + hip_attention_decode_bf16 in three launches instead of four: the norm, the rotation and the
 * cache append ride in the launch that computes the scores; every rounding point of the reference is kept (BF16 q, k,
 * scores and probabilities, cccc/MatrixEx.cpp:3018-3104, cccc-hip/hip_functions.cpp:776-804).  Arguments as
 * hip_attention_decode_fused_bf16. */
C_EXPORT int hip_attention_decode_exact_bf16(const void* q, const void* k, const void* v,
                                             const void* q_norm_w, const void* k_norm_w,
                                             const void* cos_tab, const void* sin_tab,
                                             void* k_cache, void* v_cache, void* y,
                                             void* workspace, unsigned long long workspace_bytes,
                                             int n_q_heads, int n_kv_heads, int head_dim, int t_kv,
                                             const void* d_pos, float epsilon);

/*
 * The same neighbours for a whole prompt: T tokens at positions pos0 .. pos0 + T - 1 in one pass (what the reference's graph
 * does when cccc-llm feeds it T tokens at once, cccc-llm/cccc-llm.cpp:589-618), between hip_quant_gemm calls with T columns.
 * Activations are token-major BF16 ([T][features], i.e. the column-major [features x T] hip_quant_gemm writes).
 */

/* Per-head RMSNorm (NULL, NULL: none) and RoPE of q [T][n_q_heads][128] and k [T][n_kv_heads][128] at table rows
 * pos0 + t; q_out as q; k and v [T][n_kv_heads][128] go to rows pos0 + t of the caches ([kv_head][t_kv][128]). */
C_EXPORT int hip_qk_norm_rope_kv_rows_bf16(const void* q, const void* k, const void* v,
                                           const void* q_norm_w, const void* k_norm_w,
                                           const void* cos_tab, const void* sin_tab,
                                           void* q_out, void* k_cache, void* v_cache,
                                           int n_q_heads, int n_kv_heads, int head_dim, int t_kv,
                                           int n_tokens, int pos0, float epsilon);

/* Causal GQA attention of the T rotated queries q [T][n_q_heads][128] over cache rows 0 .. pos0 + t (rows pos0 .. pos0 + T - 1
 * already appended): scores rounded to BF16, keys past the token's position masked, FP32 softmax over the row, BF16
 * probabilities, y [T][n_q_heads][128] = bf16(V p) -- the rounding points of cccc/MatrixEx.cpp:3018-3104.  On the matrix
 * cores; no workspace.  n_q_heads / n_kv_heads must be 1, 2 or 4. */
C_EXPORT int hip_attention_prefill_bf16(const void* q, const void* k_cache, const void* v_cache, void* y,
                                        int n_q_heads, int n_kv_heads, int head_dim, int t_kv,
                                        int n_tokens, int pos0);

/* y = bf16(a + b) and y = bf16(bf16(gate * bf16(sigmoid(gate))) * up) over n BF16 elements (n % 8 == 0, 16-byte aligned):
 * the residual add and the SwiGLU product with the reference's roundings (cccc-hip/hip_functions.cpp:895-908, :722-732,
 * :953-966; cccc/MatrixEx.cpp:756-762). */
C_EXPORT int hip_add_bf16(const void* a, const void* b, void* y, unsigned long long n);
C_EXPORT int hip_swiglu_bf16(const void* gate, const void* up, void* y, unsigned long long n);

/* Up to three linears on the same activations in one launch: Y[s][t][o] = bf16(W[s] x_t), s < n_segments <= 3, FP8 weights
 * [n_out[s]][K] of one type, K and row pitch ldw (all on their registered tiled copies, or all on the file layout), BF16
 * activations [tokens][K] and outputs with row pitch ldy[s] -- the q, k and v projections of a prompt, whose narrow members
 * alone leave most of the GPU idle.  With too few output tiles for the GPU (FP8, K >= 1024) the k range is split over
 * workgroups, the FP32 partial sums go to a workspace the library grows on demand and one more launch adds them for all
 * segments; otherwise the bits of the separate hip_quant_gemm calls (alpha 1, beta 0) where those do not split either.
 * FP4 block-scale weights (type 6) take part when every one has a registered tiled copy of one block length and K is a
 * multiple of 128.  -1 (nothing launched): other weight types, fewer than 2 tokens, K not a multiple of 64.  No counterpart
 * in the reference, which issues one batchedMul per projection (scripts/convert_weights.py:492-500). */
C_EXPORT int hip_quant_gemm_segments(int n_segments, const int* n_out, const void* const* W, const float* inv_scale,
                                     void* const* Y, const int* ldy, int w_type, int tokens, int K, int ldw, const void* X, int ldx);

/* A linear, the residual add behind it and the RMSNorm behind that, for the shapes whose GEMM splits its k range over
 * workgroups (few output tiles: the o and down projections of a prompt of up to ~512 tokens): sum[t] = bf16(res[t] +
 * bf16(W x_t)), y[t] = rmsnorm(sum[t]) * norm_w -- the launch that adds the FP32 partial sums does the add and the norm as
 * well, with the bits of hip_quant_gemm + hip_add_bf16 + hip_rms_norm_fwd (hip_functions.cpp:895-908, :1121-1160).  FP8
 * weights [n_out][K] (row pitch ldw; tiled copy used when registered) or FP4 block-scale weights with a registered tiled copy
 * (K % 128 == 0, ldw == K); BF16 activations [tokens][K]; res, sum, y dense [tokens][n_out], n_out <= 4096 and a multiple
 * of 8, everything 16-byte aligned.  -1 (nothing launched, use the separate calls): a shape that does not split, fewer than
 * 2 tokens, anything else unsupported.  No counterpart in the reference. */
C_EXPORT int hip_quant_gemm_add_rms_norm(int n_out, int tokens, int K, const void* W, int w_type, int ldw, float inv_scale,
                                         const void* X, int ldx, const void* res, void* sum, const void* norm_w, void* y, float epsilon);

/* y[t][o] = swiglu(gate[t][o], up[t][o]) with gate = bf16(W_gate x_t), up = bf16(W_up x_t): the gate and up linears of an
 * MLP block (two FP8 weights of one shape [n_out][K], row pitch ldw, dequantisation multipliers as in hip_quant_gemm; both
 * on their registered tiled copies or both on the file layout) and the reference's SwiGLU product
 * bf16(bf16(g * bf16(sigmoid g)) * u) (cccc/MatrixEx.cpp:756-762, hip_functions.cpp:722-732, :953-966) in one launch, with
 * the bits of the three calls it replaces -- or, with too few output tiles for the GPU (K >= 1024), the k range split over
 * workgroups and a second launch that adds the FP32 partial sums (workspace grown on demand) and writes the product with
 * the same roundings.  BF16 activations [tokens][K] (row pitch ldx) and output [tokens][n_out] (ldy).  FP4 block-scale
 * weights (type 6) take part when both have a registered tiled copy of one block length, K is a multiple of 128 and
 * ldw == K.  -1 (nothing launched, use the separate calls): other weight types, fewer than 2 tokens, K not a multiple of 64.
 * (Up to 16 tokens the separate calls are matrix-vector kernels; on the file layout the fused launches are ahead from about
 * 5 tokens on, on tiled copies from 17.) */
C_EXPORT int hip_quant_gemm_swiglu(int n_out, int tokens, int K, const void* W_gate, const void* W_up, int w_type, int ldw,
                                   float inv_scale_gate, float inv_scale_up, const void* X, int ldx, void* Y, int ldy);

/* sum = bf16(a + b) and y = rmsnorm(sum) * norm_w, rows of `inner` BF16 values (a multiple of 8, at most 4096; 16-byte
 * aligned pointers, else -1): hip_add_bf16 followed by hip_rms_norm_fwd in one pass, the same bits.  `sum` and `y` are
 * buffers of their own.  The residual add and the norm behind it in the reference's graph (hip_functions.cpp:895-908, :1506-1535). */
C_EXPORT int hip_add_rms_norm_bf16(const void* a, const void* b, void* sum, const void* norm_w, void* y,
                                   unsigned int rows, unsigned int inner, float epsilon);

/* Embedding row of token *d_token (int32 in device memory) -> y bf16 [D]. */
C_EXPORT int hip_embed_token_bf16(const void* d_token, const void* W, void* y, int D, int n_rows);

/* Arg-max of n BF16 values (lowest index on ties) into *d_index (int32, device); when d_pos is not
 * NULL, *d_pos is incremented afterwards (the step counter of a decode loop).  `workspace`:
 * hip_argmax_workspace_bytes(n) bytes of device memory for the per-block candidates. */
C_EXPORT unsigned long long hip_argmax_workspace_bytes(unsigned int n);
C_EXPORT int hip_argmax_bf16(const void* x, unsigned int n, void* d_index, void* d_pos, void* workspace);
/* The same pick in one launch from the candidate list a hip_quant_linear_fused launch left in `workspace`
 * (its argmax_workspace; n = that launch's n_out[0]) -- the reference does this on the host after copying the
 * logits back (cccc-llm/cccc-llm.cpp:546).  When embed_W is not NULL the launch also copies row *d_index of the
 * BF16 table embed_W [n_rows][D] to embed_y: the embedding of the next step. */
C_EXPORT int hip_argmax_pick_embed_bf16(const void* workspace, unsigned int n, void* d_index, void* d_pos,
                                        const void* embed_W, void* embed_y, int D, int n_rows);

/*
 * Library controls (no counterpart in the reference, which always uses the null stream and always
 * synchronises: cccc-hip/hip_functions.cpp:32-42).
 * Both switches are per host thread, like the reference's current-device pointer (cccc/GpuControl.cpp:18);
 * the library is meant to be driven by one host thread per device, as the reference drives its own.
 *   hip_quant_set_sync(1)   : hipDeviceSynchronize + error check after every launch of this thread
 *                             (parity/debug); returns the previous setting
 *   hip_quant_set_stream(s) : this thread's launches go to hipStream_t `s` (NULL = null stream)
 *   hip_quant_get_stream()  : the hipStream_t this thread's launches currently go to (NULL = null stream), for a
 *                             caller that has copies of its own to order with them
 *   hip_quant_last_kernel() : name of the kernel family the last hip_quant_gemm call dispatched to
 *                             ("gemv_dot2", "gemv_mfma", "gemm_mfma", "generic", ...)
 */
/*
 * Workspace of the k-split launches (no counterpart in the reference, whose grow-only workspaces live in its BLAS
 * wrapper, cccc/cublas_real.h:1174-1225).  A GEMM whose output has too few tiles for the GPU splits K over workgroups and
 * keeps FP32 partial sums in a buffer per (host thread, device, stream) that grows on demand and lives until the process
 * ends.  The buffer is never grown while the stream is being captured into a graph: a call that would need a larger one
 * then runs without the split (hip_quant_gemm, hip_quant_gemm_segments, hip_quant_gemm_swiglu: same result up to the FP32
 * summation order) or returns -1 (hip_quant_gemm_add_rms_norm).  A caller that captures such launches either runs each
 * shape once eagerly on the same stream first, or reserves the bytes up front with
 *   hip_quant_workspace_reserve(bytes) : grows this thread's buffer for the current device and stream to at least
 *                                        `bytes` (16 * tokens * n_out * 4 covers every split; a gate / up pair twice that).
 *                                        0 ok, 1 allocation failed, -1 the stream is being captured.
 */
C_EXPORT int hip_quant_workspace_reserve(unsigned long long bytes);

C_EXPORT int hip_quant_set_sync(int enabled);
C_EXPORT int hip_quant_set_stream(void* stream);
C_EXPORT void* hip_quant_get_stream(void);
C_EXPORT const char* hip_quant_last_kernel(void);
