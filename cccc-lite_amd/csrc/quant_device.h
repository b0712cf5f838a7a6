// Device-side scalar formats and wave64 helpers shared by the gfx950 kernels.
//
// Decoders follow the reference bit for bit:
//   E5M2  cccc/types.h:139-166, cccc-cuda/cuda_functions.cu:2674-2693
//   E4M3  cccc/types.h:72-90,   cccc-cuda/cuda_functions.cu:2366-2381
//   FP4   cccc/types.h:208-216, cccc-cuda/cuda_functions.cu:2791-2794
//   BF16 rounding: cccc-cuda/cuda_functions.cu:2761-2764
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ccq
{

enum DataType : int
{
    DT_FLOAT = 0,
    DT_DOUBLE = 1,
    DT_HALF = 2,
    DT_BF16 = 3,
    DT_E4M3 = 4,
    DT_E5M2 = 5,
    DT_FP4 = 6,
};

typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

__device__ __forceinline__ float bits_to_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f32_to_bits(float f) { return __builtin_bit_cast(uint32_t, f); }

// ---- exact software decoders (used where the result must equal the reference bit for bit)

__device__ __forceinline__ float e5m2_to_f32(uint32_t b)
{
    const uint32_t sign = (b & 0x80u) << 24;
    const uint32_t e = (b >> 2) & 31u;
    const uint32_t m = b & 3u;
    if (e == 31u) { return bits_to_f32(m ? 0x7FC00000u : (sign | 0x7F800000u)); }
    if (e == 0u)
    {
        const float mag = (float)m * (1.0f / 65536.0f);
        return bits_to_f32(f32_to_bits(mag) | sign);
    }
    return bits_to_f32(sign | ((e + 112u) << 23) | (m << 21));
}

__device__ __forceinline__ float e4m3_to_f32(uint32_t b)
{
    const uint32_t sign = (b & 0x80u) << 24;
    const uint32_t e = (b >> 3) & 15u;
    const uint32_t m = b & 7u;
    if (e == 15u && m == 7u) { return bits_to_f32(0x7FC00000u); }
    if (e == 0u)
    {
        const float mag = (float)m * (1.0f / 512.0f);
        return bits_to_f32(f32_to_bits(mag) | sign);
    }
    return bits_to_f32(sign | ((e + 120u) << 23) | (m << 20));
}

// magnitude = {0, .5, 1, 1.5, 2, 3, 4, 6}[n & 7], sign = bit 3; written without a table so it
// lives in registers: e = (n>>1)&3, m = n&1 -> e==0 ? m*0.5 : (1 + m/2) * 2^(e-1).
// Code 8 is +0.0 in the reference table (not -0.0), so the sign only applies to non-zero codes.
__device__ __forceinline__ float fp4_to_f32(uint32_t n)
{
    const uint32_t sign = (n & 7u) ? ((n & 8u) << 28) : 0u;
    const uint32_t e = (n >> 1) & 3u;
    const uint32_t m = n & 1u;
    const uint32_t normal = ((e + 126u) << 23) | (m << 22);
    const uint32_t sub = m ? 0x3F000000u : 0u;
    return bits_to_f32(sign | (e ? normal : sub));
}

// Round-to-nearest-even f32 -> bf16 by the reference's integer trick.
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f)
{
    uint32_t u = f32_to_bits(f);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return u >> 16;
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return bits_to_f32(h << 16); }

// Epilogue shared by every kernel: alpha / beta in FP32, one rounding to BF16.
__device__ __forceinline__ uint16_t finish_output(float acc, float alpha, float beta, const uint16_t* y)
{
    float r = alpha * acc;
    if (beta != 0.0f) { r += beta * bf16_bits_to_f32(*y); }
    return (uint16_t)f32_to_bf16_bits(r);
}

// ---- IEEE half (the reference's other 16-bit activation type, cccc/cublas_real.h:921-938)

__device__ __forceinline__ uint32_t f32_to_half_bits(float f)
{
    const _Float16 h = (_Float16)f;    // v_cvt_f16_f32, round to nearest even
    // the sign is carried over explicitly so that -0.0 stays -0.0
    return ((uint32_t)__builtin_bit_cast(uint16_t, h) & 0x7FFFu) | ((f32_to_bits(f) >> 16) & 0x8000u);
}

__device__ __forceinline__ float half_bits_to_f32(uint32_t h) { return (float)__builtin_bit_cast(_Float16, (uint16_t)h); }

// 16-bit activation / output element of type AT (DT_BF16 or DT_HALF)
template <int AT>
__device__ __forceinline__ float act_bits_to_f32(uint32_t h) { return AT == DT_HALF ? half_bits_to_f32(h) : bf16_bits_to_f32(h); }

template <int AT>
__device__ __forceinline__ uint32_t f32_to_act_bits(float f) { return AT == DT_HALF ? f32_to_half_bits(f) : f32_to_bf16_bits(f); }

template <int AT>
__device__ __forceinline__ uint16_t finish_output_act(float acc, float alpha, float beta, const uint16_t* y)
{
    float r = alpha * acc;
    if (beta != 0.0f) { r += beta * act_bits_to_f32<AT>(*y); }
    return (uint16_t)f32_to_act_bits<AT>(r);
}

// ---- wave64 reductions (DPP inside a 16-lane row, then across the four rows)

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

// Sum over the 64 lanes of a wave; every lane of row 0..3 ends with its row's sum after the DPP
// steps, the cross-row step reads lanes 0/16/32/48 back through SGPRs.  Result is wave-uniform.
__device__ __forceinline__ float wave_sum(float v)
{
    v += dpp_f32<0xB1>(v);     // quad_perm [1,0,3,2]
    v += dpp_f32<0x4E>(v);     // quad_perm [2,3,0,1]
    v += dpp_f32<0x141>(v);    // row_half_mirror
    v += dpp_f32<0x140>(v);    // row_mirror
    const int b = __builtin_bit_cast(int, v);
    const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0));
    const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
    const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32));
    const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
    return (r0 + r1) + (r2 + r3);
}

// Sum of squares of eight BF16 values (one 16-byte chunk of a row), and the chunk scaled by 1 / rms and the norm weight:
// the arithmetic of every row norm in the library, kept in one place so that the fused variants give the same bits.
__device__ __forceinline__ float sumsq8(const u32x4& v)
{
    float s = 0.0f;
#pragma unroll
    for (int d = 0; d < 4; d++)
    {
        const float lo = bf16_bits_to_f32(v[d] & 0xFFFFu), hi = bf16_bits_to_f32(v[d] >> 16);
        s += lo * lo + hi * hi;
    }
    return s;
}

__device__ __forceinline__ u32x4 normed8(const u32x4& v, const u32x4& w, float invstd)
{
    u32x4 out;
#pragma unroll
    for (int d = 0; d < 4; d++)
    {
        const float lo = bf16_bits_to_f32(v[d] & 0xFFFFu) * invstd * bf16_bits_to_f32(w[d] & 0xFFFFu);
        const float hi = bf16_bits_to_f32(v[d] >> 16) * invstd * bf16_bits_to_f32(w[d] >> 16);
        out[d] = f32_to_bf16_bits(lo) | (f32_to_bf16_bits(hi) << 16);
    }
    return out;
}


}    // namespace ccq
