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
 * with FP32 accumulation, alpha/beta applied in FP32, rounded once to BF16.  `act_scale` is
 * accepted and ignored (it only drives the W8A8 route, cccc/cublas_real.h:871-873).
 * Anything else returns -1.
 */
C_EXPORT int hip_quant_gemm(int transA, int transB, int M, int N, int K, float alpha,
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
 * (today: 5..16 tokens on tall weights such as lm_head), where the matrix-core GEMV wants the 16 rows x
 * 64 codes of one load to be contiguous.
 * Results are identical with and without it.  hip_quant_weight_release forgets the key (before the
 * caller frees either buffer).  Returns 0 ok, 1 runtime error, -1 unsupported (FP4, K % 16 != 0, ...).
 */
C_EXPORT unsigned long long hip_quant_tiled_size(int type, int n_out, int K);
C_EXPORT int hip_quant_weight_prepare(const void* W, int type, int n_out, int K, int ldw, void* dst_tiled);
C_EXPORT int hip_quant_weight_release(const void* W);

/*
 * Library controls (no counterpart in the reference, which always uses the null stream and always
 * synchronises: cccc-hip/hip_functions.cpp:32-42).
 *   hip_quant_set_sync(1)   : hipDeviceSynchronize + error check after every launch (parity/debug)
 *   hip_quant_set_stream(s) : enqueue on hipStream_t `s` (NULL = null stream)
 *   hip_quant_last_kernel() : name of the kernel family the last hip_quant_gemm call dispatched to
 *                             ("gemv_dot2", "gemv_mfma", "gemm_mfma", "generic", ...)
 */
C_EXPORT int hip_quant_set_sync(int enabled);
C_EXPORT int hip_quant_set_stream(void* stream);
C_EXPORT const char* hip_quant_last_kernel(void);
