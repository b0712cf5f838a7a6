/*
 * cccc_oracle.c -- CPU restatement of cccc's weight-only quantized linear path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker that the parity tests, the
 * smoke test and the benchmark's cpu_baseline leg compare the HIP library against.
 * Nothing in the shipped library may call, link or load it.
 *
 * Every function restates one piece of the reference (paths relative to the
 * reference tree) in plain scalar C:
 *
 *   orc_e5m2_to_float            cccc/types.h:139-166, cccc-cuda/cuda_functions.cu:2674-2693
 *   orc_e4m3_to_float            cccc/types.h:72-90,   cccc-cuda/cuda_functions.cu:2366-2381
 *   orc_fp4_to_float             cccc/types.h:208-216, cccc-cuda/cuda_functions.cu:2791-2794
 *   orc_f32_to_bf16_rne          cccc-cuda/cuda_functions.cu:2761-2764 (integer RNE trick)
 *   orc_float_to_e5m2_trunc      cccc/types.h:168-199, cccc-cuda/cuda_functions.cu:2694-2724
 *   orc_float_to_e4m3_trunc      cccc/types.h:92-123,  cccc-cuda/cuda_functions.cu:2382-2412
 *   orc_float_to_fp4             cccc/types.h:218-254, cccc-cuda/cuda_functions.cu:2796-2832
 *   orc_convert                  cccc-cuda/cuda_functions.cu:3066-3090 (dispatch table) and the
 *                                per-pair kernels it names (:53-131, :2413-2445, :2559-2596,
 *                                :2725-2785, :2834-2884)
 *   orc_fp4_blockscale_to_bf16   cccc-cuda/cuda_functions.cu:2926-2939, :2953-2960
 *   orc_float_to_fp4_blockscale  cccc-cuda/cuda_functions.cu:2896-2923, :2943-2950
 *   orc_quant_gemm               cccc/cublas_real.h:875-881, :943-964, :1066-1087 (dequantize the
 *                                whole quantized operand to a BF16 workspace, then a BF16 GEMM with
 *                                FP32 accumulation, alpha/beta in FP32, one rounding to BF16)
 *   orc_cpu_linear               cccc/Matrix.cpp:1258-1267 -> cccc/cblas_real.h:332-334: the
 *                                reference CPU path (whole-weight dequant to f32 + cblas_sgemm)
 *
 * Pinning status (what independent evidence each decoder is checked against in tests/):
 *   e5m2 / e4m3 decode : torch.float8_e5m2 / torch.float8_e4m3fn -> float32 on all non-NaN codes;
 *                        "E5M2 = high byte of IEEE fp16"; the reference's own cccc/types.h compiled
 *                        as oracle/_ref (all 256 codes incl. NaN canonicalisation).
 *   fp4 decode         : 16-entry literal table; oracle/_ref.
 *   bf16 rounding      : torch .to(bfloat16) (RNE) over an exhaustive code x scale sweep.
 *   encoders (trunc)   : oracle/_ref (cccc/types.h host encoders) on a dense sweep + brute force.
 *   GEMM               : cuBLAS/OpenBLAS are not in the reference tree and the reference has no
 *                        test vectors for it -- PARITY UNPINNED by the reference; pinned instead
 *                        against exact (float64) contraction of the bit-exact dequantized weights,
 *                        one-hot / all-ones activations and numpy matmul.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

/* cccc::DataType values (cccc/types.h:24-34) */
enum { ORC_FLOAT = 0, ORC_DOUBLE = 1, ORC_HALF = 2, ORC_BF16 = 3, ORC_E4M3 = 4, ORC_E5M2 = 5, ORC_FP4 = 6 };

static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* ------------------------------------------------------------------ decoders */

float orc_e5m2_to_float(uint8_t b)
{
    uint32_t sign = (uint32_t)(b >> 7);
    uint32_t e = (b >> 2) & 31u;
    uint32_t m = b & 3u;
    if (e == 31u)
        return m ? bits_f32(0x7FC00000u)                     /* every NaN code -> +qNaN, sign dropped */
                 : bits_f32((sign << 31) | 0x7F800000u);     /* +-Inf */
    if (e == 0u)
        return (sign ? -1.0f : 1.0f) * (float)m * (1.0f / 65536.0f);
    return bits_f32((sign << 31) | ((e + 112u) << 23) | (m << 21));
}

float orc_e4m3_to_float(uint8_t b)
{
    uint32_t sign = (uint32_t)(b >> 7);
    uint32_t e = (b >> 3) & 15u;
    uint32_t m = b & 7u;
    if (e == 15u && m == 7u)
        return bits_f32(0x7FC00000u);
    if (e == 0u)
        return (sign ? -1.0f : 1.0f) * (float)m * (1.0f / 512.0f);
    return bits_f32((sign << 31) | ((e + 120u) << 23) | (m << 20));
}

static const float k_fp4_values[16] = { 0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f,
                                        0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f };

float orc_fp4_to_float(uint8_t nibble) { return k_fp4_values[nibble & 15u]; }

/* element i of a packed nibble buffer: low nibble holds the even element */
static inline uint8_t fp4_nibble_at(const uint8_t* bytes, size_t i)
{
    uint8_t byte = bytes[i >> 1];
    return (i & 1u) ? (uint8_t)(byte >> 4) : (uint8_t)(byte & 15u);
}

/* ------------------------------------------------------------------ roundings */

uint16_t orc_f32_to_bf16_rne(float f)
{
    uint32_t u = f32_bits(f);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

float orc_bf16_to_float(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* IEEE binary16 <-> binary32, round to nearest even (what __float2half_rn / __half2float do) */
uint16_t orc_f32_to_half_rne(float f)
{
    uint32_t u = f32_bits(f);
    uint32_t sign = (u >> 16) & 0x8000u;
    uint32_t mag = u & 0x7FFFFFFFu;
    if (mag > 0x7F800000u) return (uint16_t)(sign | 0x7E00u | ((mag >> 13) & 0x1FFu)); /* NaN */
    if (mag >= 0x47800000u) return (uint16_t)(sign | 0x7C00u);                         /* >= 65536 -> Inf (incl. Inf) */
    if (mag < 0x33000000u) return (uint16_t)sign;                                      /* < 2^-25 -> 0 */
    int32_t exp = (int32_t)(mag >> 23) - 127;
    uint32_t man = (mag & 0x7FFFFFu) | 0x800000u;
    uint32_t shift = (exp < -14) ? (uint32_t)(13 + (-14 - exp)) : 13u;
    uint32_t kept = man >> shift;
    uint32_t rest = man & ((1u << shift) - 1u);
    uint32_t half_ulp = 1u << (shift - 1u);
    if (rest > half_ulp || (rest == half_ulp && (kept & 1u))) kept++;
    uint32_t out;
    if (exp < -14) out = kept;                                   /* subnormal (may carry into normal) */
    else           out = ((uint32_t)(exp + 15) << 10) + (kept - 0x400u);
    return (uint16_t)(sign | out);                               /* carry into exponent/Inf is correct */
}

float orc_half_to_float(uint16_t h)
{
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 31u;
    uint32_t m = h & 0x3FFu;
    if (e == 31u) return bits_f32(sign | 0x7F800000u | (m << 13));
    if (e == 0u) {
        float v = (float)m * (1.0f / 16777216.0f);               /* m * 2^-24 */
        return sign ? -v : v;
    }
    return bits_f32(sign | ((e + 112u) << 23) | (m << 13));
}

/* ------------------------------------------------------------------ encoders */

/* Truncating (round-toward-zero) float -> E5M2 of the reference; saturates to 0x7B. */
uint8_t orc_float_to_e5m2_trunc(float f, float scale)
{
    f *= scale;
    uint32_t u = f32_bits(f);
    uint32_t mag = u & 0x7FFFFFFFu;
    uint32_t sign = u >> 31;
    if (mag > 0x7F800000u) return 0x7Cu;
    if (mag == 0x7F800000u) return (uint8_t)((sign << 7) | 0x7Cu);
    int fe = (int)((u >> 23) & 255u) - 127;
    uint32_t fm = u & 0x7FFFFFu;
    if (fe > 15 || (fe == 15 && fm >= 0xE00000u)) return (uint8_t)((sign << 7) | 0x7Bu);
    int e8 = fe + 15;
    if (e8 <= 0) {
        int shift = 7 - fe;
        if (shift >= 32) return (uint8_t)(sign << 7);
        return (uint8_t)((sign << 7) | (((fm | 0x800000u) >> shift) & 3u));
    }
    return (uint8_t)((sign << 7) | ((uint32_t)(e8 & 31) << 2) | (fm >> 21));
}

/* Truncating float -> E4M3 of the reference; saturates to 0x7E (448), NaN -> 0x7F. */
uint8_t orc_float_to_e4m3_trunc(float f, float scale)
{
    f *= scale;
    uint32_t u = f32_bits(f);
    uint32_t sign = u >> 31;
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0x7Fu;
    int fe = (int)((u >> 23) & 255u) - 127;
    uint32_t fm = u & 0x7FFFFFu;
    if (fe > 8 || (fe == 8 && fm >= 0xC00000u)) return (uint8_t)((sign << 7) | 0x7Eu);
    int e8 = fe + 7;
    if (e8 <= 0) {
        int shift = 14 - fe;
        if (shift >= 32) return (uint8_t)(sign << 7);
        return (uint8_t)((sign << 7) | (((fm | 0x800000u) >> shift) & 7u));
    }
    uint32_t m8 = fm >> 20;
    if (e8 == 15 && m8 == 7u) m8 = 6u;
    return (uint8_t)((sign << 7) | ((uint32_t)(e8 & 15) << 3) | m8);
}

/* Threshold float -> E2M1 nibble of the reference (boundary value goes to the upper code). */
uint8_t orc_float_to_fp4(float f)
{
    static const float upper[7] = { 0.25f, 0.75f, 1.25f, 1.75f, 2.5f, 3.5f, 5.0f };
    uint8_t s = (f < 0.0f) ? 8u : 0u;
    float a = (f < 0.0f) ? -f : f;
    uint8_t code = 7u;
    for (int i = 0; i < 7; i++)
        if (a < upper[i]) { code = (uint8_t)i; break; }
    return (uint8_t)(s | code);
}

/* Our own synthetic-data encoder: float -> E5M2 with round-to-nearest-even (IEEE semantics,
 * overflow to Inf).  Not a reference function: the reference only truncates.  E5M2 is the high
 * byte of binary16 with 8 fewer mantissa bits, so: round f32 -> f16 (RNE) is NOT equivalent
 * (double rounding); instead round the f32 mantissa directly at 2 bits. */
uint8_t orc_float_to_e5m2_rne(float f)
{
    uint32_t u = f32_bits(f);
    uint32_t sign = (u >> 24) & 0x80u;
    uint32_t mag = u & 0x7FFFFFFFu;
    if (mag > 0x7F800000u) return (uint8_t)(sign | 0x7Fu);
    if (mag >= 0x47800000u) return (uint8_t)(sign | 0x7Cu);   /* >= 65536 (incl. Inf) */
    if (mag <= 0x37000000u) return (uint8_t)sign;             /* <= 2^-17: ties-to-even at half the smallest subnormal -> 0 */
    int32_t exp = (int32_t)(mag >> 23) - 127;
    uint32_t man = (mag & 0x7FFFFFu) | 0x800000u;
    uint32_t shift = (exp < -14) ? (uint32_t)(21 + (-14 - exp)) : 21u;
    uint32_t kept = man >> shift;
    uint32_t rest = man & ((1u << shift) - 1u);
    uint32_t half_ulp = 1u << (shift - 1u);
    if (rest > half_ulp || (rest == half_ulp && (kept & 1u))) kept++;
    uint32_t out = (exp < -14) ? kept : (((uint32_t)(exp + 15) << 2) + (kept - 4u));
    return (uint8_t)(sign | out);                             /* 0x7C on carry = Inf, as IEEE */
}

/* ------------------------------------------------------------------ convert */

static float load_as_float(const void* src, int type, size_t i)
{
    switch (type) {
    case ORC_FLOAT: return ((const float*)src)[i];
    case ORC_HALF:  return orc_half_to_float(((const uint16_t*)src)[i]);
    case ORC_BF16:  return orc_bf16_to_float(((const uint16_t*)src)[i]);
    case ORC_E4M3:  return orc_e4m3_to_float(((const uint8_t*)src)[i]);
    case ORC_E5M2:  return orc_e5m2_to_float(((const uint8_t*)src)[i]);
    case ORC_FP4:   return orc_fp4_to_float(fp4_nibble_at((const uint8_t*)src, i));
    default:        return 0.0f;
    }
}

/* Which (src,dst) pairs the reference table fills, and whether that pair's kernel uses `scale`. */
static int convert_pair_supported(int s, int d, int* uses_scale)
{
    *uses_scale = 0;
    if (s == ORC_FLOAT && d == ORC_BF16) return 1;
    if (s == ORC_FLOAT && (d == ORC_E4M3 || d == ORC_E5M2 || d == ORC_FP4)) { *uses_scale = 1; return 1; }
    if (s == ORC_HALF && (d == ORC_FLOAT || d == ORC_BF16)) return 1;
    if (s == ORC_BF16 && (d == ORC_FLOAT || d == ORC_HALF)) return 1;
    if (s == ORC_BF16 && d == ORC_E4M3) { *uses_scale = 1; return 1; }
    if ((s == ORC_E4M3 || s == ORC_E5M2) && (d == ORC_FLOAT || d == ORC_HALF || d == ORC_BF16)) { *uses_scale = 1; return 1; }
    if (s == ORC_FP4 && (d == ORC_FLOAT || d == ORC_BF16)) { *uses_scale = 1; return 1; }
    return 0;
}

/* Returns 0 ok, -1 unsupported pair.  `n` counts elements, except for the same-type copy where
 * the reference copies `n` BYTES (cuda_functions.cu:3068-3072) -- kept as is. */
int orc_convert(const void* src, int src_type, void* dst, int dst_type, unsigned int n, float scale)
{
    if (src_type == dst_type && scale == 1.0f) { memmove(dst, src, (size_t)n); return 0; }
    if ((unsigned)src_type >= 7u || (unsigned)dst_type >= 7u) return -1;
    int uses_scale;
    if (!convert_pair_supported(src_type, dst_type, &uses_scale)) return -1;
    if (dst_type == ORC_FP4) {                      /* two elements per output byte */
        uint8_t* out = (uint8_t*)dst;
        for (size_t e0 = 0; e0 < n; e0 += 2) {
            uint8_t lo = orc_float_to_fp4(((const float*)src)[e0] * scale);
            uint8_t hi = (e0 + 1 < n) ? orc_float_to_fp4(((const float*)src)[e0 + 1] * scale) : 0u;
            out[e0 >> 1] = (uint8_t)(lo | (hi << 4));
        }
        return 0;
    }
    for (size_t i = 0; i < n; i++) {
        float v = load_as_float(src, src_type, i);
        switch (dst_type) {
        case ORC_FLOAT: ((float*)dst)[i] = uses_scale ? v * scale : v; break;
        case ORC_HALF:  ((uint16_t*)dst)[i] = orc_f32_to_half_rne(uses_scale ? v * scale : v); break;
        case ORC_BF16:  ((uint16_t*)dst)[i] = orc_f32_to_bf16_rne(uses_scale ? v * scale : v); break;
        case ORC_E4M3:  ((uint8_t*)dst)[i] = orc_float_to_e4m3_trunc(v, scale); break;
        case ORC_E5M2:  ((uint8_t*)dst)[i] = orc_float_to_e5m2_trunc(v, scale); break;
        default: return -1;
        }
    }
    return 0;
}

int orc_fp4_blockscale_to_bf16(const void* nibbles, const void* scales, void* dst,
                               unsigned int n_elems, unsigned int block_size)
{
    if (block_size == 0u) return -1;
    const uint8_t* nb = (const uint8_t*)nibbles;
    const uint8_t* sc = (const uint8_t*)scales;
    uint16_t* out = (uint16_t*)dst;
    for (size_t i = 0; i < n_elems; i++) {
        float s = orc_e4m3_to_float(sc[i / block_size]);
        float v = orc_fp4_to_float(fp4_nibble_at(nb, i)) * s;
        out[i] = orc_f32_to_bf16_rne(v);
    }
    return 0;
}

int orc_float_to_fp4_blockscale(const void* src, void* nibbles, void* scales,
                                unsigned int n_elems, unsigned int block_size)
{
    if (block_size == 0u) return -1;
    const float* x = (const float*)src;
    uint8_t* nb = (uint8_t*)nibbles;
    uint8_t* sc = (uint8_t*)scales;
    size_t n_blocks = ((size_t)n_elems + block_size - 1) / block_size;
    for (size_t b = 0; b < n_blocks; b++) {
        size_t lo = b * block_size, hi = lo + block_size;
        if (hi > n_elems) hi = n_elems;
        float amax = 0.0f;
        for (size_t i = lo; i < hi; i++) amax = fmaxf(amax, fabsf(x[i]));
        float fwd = (amax > 1e-10f) ? (6.0f / amax) : 1.0f;
        float dq = (amax > 1e-10f) ? (amax / 6.0f) : 1.0f;
        sc[b] = orc_float_to_e4m3_trunc(dq, 1.0f);
        for (size_t i = lo; i < hi; i += 2) {
            uint8_t l = orc_float_to_fp4(x[i] * fwd);
            uint8_t h = (i + 1 < n_elems) ? orc_float_to_fp4(x[i + 1] * fwd) : 0u;
            nb[i >> 1] = (uint8_t)(l | (h << 4));
        }
    }
    return 0;
}

/* ------------------------------------------------------------------ unified quantized GEMM */

static int is_quantized(int t) { return t == ORC_E4M3 || t == ORC_E5M2 || t == ORC_FP4; }

/* Dequantize `count` flat elements of a quantized operand to bf16 bits, the way the weight-is-A /
 * weight-is-B BF16 branches do before the GEMM (cublas_real.h:952-955, :1075-1078). */
static void dequant_operand_bf16(const void* q, int type, float inv_scale, const uint8_t* blk_sc,
                                 unsigned block_size, size_t count, uint16_t* out)
{
    if (type == ORC_FP4 && blk_sc)
        orc_fp4_blockscale_to_bf16(q, blk_sc, out, (unsigned)count, block_size);
    else
        orc_convert(q, type, out, ORC_BF16, (unsigned)count, inv_scale);
}

/*
 * Column-major C[M x N] = bf16( alpha * op(A)[M x K] * op(B)[K x N] + beta * C ), with exactly one
 * of A / B quantized and the other BF16, C BF16 (the W8A16 / FP4 BF16 branches).
 * trans flags: 0 = no-trans, 1 = trans (MatrixTransType).  acc64 != 0 accumulates in double (the
 * "exact" value tests compare against); acc64 == 0 accumulates sequentially in float.
 * Returns 0 ok, -1 for a type combination outside those branches.
 */
int orc_quant_gemm(int transA, int transB, int M, int N, int K, float alpha,
                   const void* A, int typeA, int lda, float invScaleA,
                   const void* B, int typeB, int ldb, float invScaleB,
                   float beta, void* C, int typeC, int ldc,
                   const uint8_t* blk_scA, const uint8_t* blk_scB, unsigned block_size, int acc64)
{
    int aQ = is_quantized(typeA), bQ = is_quantized(typeB);
    if (aQ == bQ || typeC != ORC_BF16) return -1;
    if ((aQ && typeB != ORC_BF16) || (bQ && typeA != ORC_BF16)) return -1;
    size_t szA = (size_t)lda * (size_t)(transA ? M : K);
    size_t szB = (size_t)ldb * (size_t)(transB ? K : N);
    uint16_t* ws = NULL;
    const uint16_t* a16 = (const uint16_t*)A;
    const uint16_t* b16 = (const uint16_t*)B;
    if (aQ) {
        ws = (uint16_t*)malloc(szA * 2 + 2);
        dequant_operand_bf16(A, typeA, invScaleA, blk_scA, block_size, szA, ws);
        a16 = ws;
    } else {
        ws = (uint16_t*)malloc(szB * 2 + 2);
        dequant_operand_bf16(B, typeB, invScaleB, blk_scB, block_size, szB, ws);
        b16 = ws;
    }
    uint16_t* c16 = (uint16_t*)C;
    for (int n = 0; n < N; n++) {
        for (int m = 0; m < M; m++) {
            double accd = 0.0;
            float accf = 0.0f;
            for (int k = 0; k < K; k++) {
                size_t ia = transA ? ((size_t)k + (size_t)m * lda) : ((size_t)m + (size_t)k * lda);
                size_t ib = transB ? ((size_t)n + (size_t)k * ldb) : ((size_t)k + (size_t)n * ldb);
                float av = orc_bf16_to_float(a16[ia]);
                float bv = orc_bf16_to_float(b16[ib]);
                if (acc64) accd += (double)av * (double)bv;
                else       accf += av * bv;
            }
            size_t ic = (size_t)m + (size_t)n * ldc;
            float r;
            if (acc64) {
                double v = (double)alpha * accd;
                if (beta != 0.0f) v += (double)beta * (double)orc_bf16_to_float(c16[ic]);
                r = (float)v;
            } else {
                r = alpha * accf;
                if (beta != 0.0f) r += beta * orc_bf16_to_float(c16[ic]);
            }
            c16[ic] = orc_f32_to_bf16_rne(r);
        }
    }
    free(ws);
    return 0;
}

/* ------------------------------------------------------------------ reference CPU path (baseline) */

typedef void (*orc_sgemm_fn)(int order, int transA, int transB, int M, int N, int K, float alpha,
                             const float* A, int lda, const float* B, int ldb, float beta,
                             float* C, int ldc);

static double now_s(void)
{
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

/* Blocked fallback SGEMM for C[n_out x tokens] = W^T X when no BLAS library can be found:
 * W f32 [n_out][K] K-contiguous, X f32 [tokens][K], Y f32 column-major ldc = n_out. */
static void fallback_sgemm_tn(int n_out, int tokens, int K, const float* W, const float* X, float* Y)
{
#pragma omp parallel for schedule(static)
    for (int o = 0; o < n_out; o++) {
        const float* w = W + (size_t)o * K;
        for (int t = 0; t < tokens; t++) {
            const float* x = X + (size_t)t * K;
            float s0 = 0, s1 = 0, s2 = 0, s3 = 0;
            int k = 0;
            for (; k + 4 <= K; k += 4) { s0 += w[k] * x[k]; s1 += w[k+1] * x[k+1]; s2 += w[k+2] * x[k+2]; s3 += w[k+3] * x[k+3]; }
            for (; k < K; k++) s0 += w[k] * x[k];
            Y[(size_t)o + (size_t)t * n_out] = (s0 + s1) + (s2 + s3);
        }
    }
}

/*
 * The reference CPU route for one quantized linear: dequantize the whole weight to f32 with the
 * scalar decoders, cblas_sgemm(ColMajor, Trans, NoTrans, n_out, tokens, K, 1, Wf, K, Xf, K, 0, Y,
 * n_out), round Y to bf16.  `sgemm` may be NULL (built-in fallback).  threads > 1 parallelises the
 * dequant loop with OpenMP.  Times (seconds) are returned in t_dequant / t_gemm.
 * W: quantized [n_out][K]; X: bf16 [tokens][K]; Y: bf16 column-major [n_out x tokens].
 */
int orc_cpu_linear(const void* W, int w_type, float inv_scale, const uint8_t* blk_sc, unsigned block_size,
                   const uint16_t* X, uint16_t* Y, int n_out, int tokens, int K,
                   orc_sgemm_fn sgemm, int threads, double* t_dequant, double* t_gemm)
{
    size_t cnt = (size_t)n_out * (size_t)K;
    float* Wf = (float*)malloc(cnt * sizeof(float));
    float* Xf = (float*)malloc((size_t)tokens * K * sizeof(float));
    float* Yf = (float*)malloc((size_t)n_out * tokens * sizeof(float));
    if (!Wf || !Xf || !Yf) { free(Wf); free(Xf); free(Yf); return 1; }
    for (size_t i = 0; i < (size_t)tokens * K; i++) Xf[i] = orc_bf16_to_float(X[i]);
    (void)threads;
    double t0 = now_s();
    const uint8_t* wb = (const uint8_t*)W;
    if (w_type == ORC_FP4 && blk_sc) {
#pragma omp parallel for schedule(static) num_threads(threads)
        for (long long i = 0; i < (long long)cnt; i++)
            Wf[i] = orc_fp4_to_float(fp4_nibble_at(wb, (size_t)i)) * orc_e4m3_to_float(blk_sc[(size_t)i / block_size]);
    } else if (w_type == ORC_E5M2) {
#pragma omp parallel for schedule(static) num_threads(threads)
        for (long long i = 0; i < (long long)cnt; i++) Wf[i] = orc_e5m2_to_float(wb[i]) * inv_scale;
    } else if (w_type == ORC_E4M3) {
#pragma omp parallel for schedule(static) num_threads(threads)
        for (long long i = 0; i < (long long)cnt; i++) Wf[i] = orc_e4m3_to_float(wb[i]) * inv_scale;
    } else if (w_type == ORC_FP4) {
#pragma omp parallel for schedule(static) num_threads(threads)
        for (long long i = 0; i < (long long)cnt; i++) Wf[i] = orc_fp4_to_float(fp4_nibble_at(wb, (size_t)i)) * inv_scale;
    } else { free(Wf); free(Xf); free(Yf); return -1; }
    double t1 = now_s();
    if (sgemm) sgemm(102 /*CblasColMajor*/, 112 /*CblasTrans*/, 111 /*CblasNoTrans*/, n_out, tokens, K,
                     1.0f, Wf, K, Xf, K, 0.0f, Yf, n_out);
    else       fallback_sgemm_tn(n_out, tokens, K, Wf, Xf, Yf);
    double t2 = now_s();
    for (size_t i = 0; i < (size_t)n_out * tokens; i++) Y[i] = orc_f32_to_bf16_rne(Yf[i]);
    if (t_dequant) *t_dequant = t1 - t0;
    if (t_gemm) *t_gemm = t2 - t1;
    free(Wf); free(Xf); free(Yf);
    return 0;
}

/* bulk helpers so Python never loops per element */
void orc_decode_table(int type, float* out256)
{
    for (int b = 0; b < 256; b++)
        out256[b] = (type == ORC_E5M2) ? orc_e5m2_to_float((uint8_t)b)
                  : (type == ORC_E4M3) ? orc_e4m3_to_float((uint8_t)b)
                  : orc_fp4_to_float((uint8_t)b);
}

void orc_encode_e5m2_rne_bulk(const float* src, uint8_t* dst, size_t n)
{
    for (size_t i = 0; i < n; i++) dst[i] = orc_float_to_e5m2_rne(src[i]);
}

/* ------------------------------------------------------------------ decode-step helpers */

/* RoPE tables as the reference's graph builds them on the host (cccc/NetCifa.cpp:431-475): float32
 * angle = t * powf(base, -2.0f * d / d_head), cosf / sinf, stored to BF16 by TRUNCATION (the host
 * bfloat16(float) constructor drops the low 16 bits, cccc/types.h:43-48).  Layout [T][d_head / 2]. */
void orc_rope_tables(int T, int d_head, float base, uint16_t* cos_out, uint16_t* sin_out)
{
    const int half = d_head / 2;
    for (int t = 0; t < T; t++) {
        for (int d = 0; d < half; d++) {
            float angle = (float)t * powf(base, -2.0f * (float)d / (float)d_head);
            cos_out[(size_t)t * half + d] = (uint16_t)(f32_bits(cosf(angle)) >> 16);
            sin_out[(size_t)t * half + d] = (uint16_t)(f32_bits(sinf(angle)) >> 16);
        }
    }
}
