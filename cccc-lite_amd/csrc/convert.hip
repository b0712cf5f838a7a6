// hip_convert / hip_fp4_blockscale_to_bf16 / hip_float_to_fp4_blockscale for gfx950.
//
// The dequantisation pairs (FP8/FP4 -> BF16/FP32/FP16) are HBM-bound streams: each lane moves
// 16 source bytes per step with one 128-bit load and writes its results with 128-bit stores,
// and the grid is a fixed multiple of the CU count walking the buffer with a grid stride.
// Numerics follow the reference kernels element for element (decode, one FP32 multiply by the
// scale, integer round-to-nearest-even to BF16): cccc-cuda/cuda_functions.cu:2566-2596 (E4M3),
// :2735-2785 (E5M2), :2834-2884 (FP4), :2896-2960 (FP4 block scale), :3066-3090 (dispatch).
#include "../../include/cccc_hip_quant.h"
#include "quant_device.h"
#include "runtime.h"
#include <hip/hip_fp16.h>

using namespace ccq;

namespace
{

constexpr int kThreads = 256;

inline unsigned grid_for(size_t work_items)
{
    const size_t want = (work_items + kThreads - 1) / kThreads;
    const size_t cap = (size_t)cu_count() * 16;
    return (unsigned)(want < 1 ? 1 : (want > cap ? cap : want));
}

template <int SRC>
__device__ __forceinline__ float decode8(uint32_t b)
{
    return SRC == DT_E5M2 ? e5m2_to_f32(b) : e4m3_to_f32(b);
}

template <int DST>
__device__ __forceinline__ void store_one(void* dst, size_t i, float v)
{
    if (DST == DT_FLOAT) { ((float*)dst)[i] = v; }
    else if (DST == DT_HALF) { ((uint16_t*)dst)[i] = (uint16_t)f32_to_half_bits(v); }
    else { ((uint16_t*)dst)[i] = (uint16_t)f32_to_bf16_bits(v); }
}

// 16 consecutive results starting at element i0 (i0 % 16 == 0, dst suitably aligned)
template <int DST>
__device__ __forceinline__ void store_sixteen(void* dst, size_t i0, const float (&v)[16])
{
    if (DST == DT_FLOAT)
    {
        f32x4* out = (f32x4*)((float*)dst + i0);
#pragma unroll
        for (int q = 0; q < 4; q++) { out[q] = f32x4{ v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3] }; }
    }
    else
    {
        uint32_t p[8];
#pragma unroll
        for (int j = 0; j < 8; j++)
        {
            const uint32_t lo = DST == DT_HALF ? f32_to_half_bits(v[2 * j]) : f32_to_bf16_bits(v[2 * j]);
            const uint32_t hi = DST == DT_HALF ? f32_to_half_bits(v[2 * j + 1]) : f32_to_bf16_bits(v[2 * j + 1]);
            p[j] = lo | (hi << 16);
        }
        u32x4* out = (u32x4*)((uint16_t*)dst + i0);
        out[0] = u32x4{ p[0], p[1], p[2], p[3] };
        out[1] = u32x4{ p[4], p[5], p[6], p[7] };
    }
}

// ---- FP8 (1 byte / element) -> FP32 / FP16 / BF16

template <int SRC, int DST>
__global__ __launch_bounds__(kThreads) void dequant8_vec_kernel(const uint8_t* __restrict__ src, void* __restrict__ dst, size_t n_vec, float scale)
{
    const size_t stride = (size_t)gridDim.x * kThreads;
    for (size_t v = (size_t)blockIdx.x * kThreads + threadIdx.x; v < n_vec; v += stride)
    {
        const u32x4 w = __builtin_nontemporal_load((const u32x4*)src + v);
        float out[16];
#pragma unroll
        for (int d = 0; d < 4; d++)
        {
#pragma unroll
            for (int b = 0; b < 4; b++) { out[4 * d + b] = decode8<SRC>((w[d] >> (8 * b)) & 0xFFu) * scale; }
        }
        store_sixteen<DST>(dst, v * 16, out);
    }
}

template <int SRC, int DST>
__global__ __launch_bounds__(kThreads) void dequant8_scalar_kernel(const uint8_t* __restrict__ src, void* __restrict__ dst, size_t begin, size_t n, float scale)
{
    const size_t stride = (size_t)gridDim.x * kThreads;
    for (size_t i = begin + (size_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += stride)
    {
        store_one<DST>(dst, i, decode8<SRC>(src[i]) * scale);
    }
}

template <int SRC, int DST>
int launch_dequant8(const void* src, void* dst, unsigned n, float scale, const char* what)
{
    if (n == 0) { return 0; }
    const bool aligned = (((uintptr_t)src | (uintptr_t)dst) & 15u) == 0;
    const size_t n_vec = aligned ? (size_t)n / 16 : 0;
    if (n_vec) { dequant8_vec_kernel<SRC, DST><<<grid_for(n_vec), kThreads, 0, stream()>>>((const uint8_t*)src, dst, n_vec, scale); }
    const size_t done = n_vec * 16;
    if (done < n) { dequant8_scalar_kernel<SRC, DST><<<grid_for(n - done), kThreads, 0, stream()>>>((const uint8_t*)src, dst, done, n, scale); }
    return finish(what);
}

// ---- FP4 (two elements / byte) -> FP32 / BF16, per-tensor scale or per-block E4M3 scale

// One lane handles 8 packed bytes = 16 elements.  BLOCKSCALE: elements [16 v, 16 v + 16) share one
// scale byte when block_size % 16 == 0 (checked by the launcher).
template <int DST, bool BLOCKSCALE>
__global__ __launch_bounds__(kThreads) void dequant4_vec_kernel(const uint8_t* __restrict__ src, const uint8_t* __restrict__ scales,
                                                               void* __restrict__ dst, size_t n_vec, unsigned block_size, float scale)
{
    const size_t stride = (size_t)gridDim.x * kThreads;
    for (size_t v = (size_t)blockIdx.x * kThreads + threadIdx.x; v < n_vec; v += stride)
    {
        const u32x2 w = __builtin_nontemporal_load((const u32x2*)src + v);
        const float s = BLOCKSCALE ? e4m3_to_f32(scales[(v * 16) / block_size]) : scale;
        float out[16];
#pragma unroll
        for (int d = 0; d < 2; d++)
        {
#pragma unroll
            for (int q = 0; q < 8; q++) { out[8 * d + q] = fp4_to_f32((w[d] >> (4 * q)) & 0xFu) * s; }
        }
        store_sixteen<DST>(dst, v * 16, out);
    }
}

template <int DST, bool BLOCKSCALE>
__global__ __launch_bounds__(kThreads) void dequant4_scalar_kernel(const uint8_t* __restrict__ src, const uint8_t* __restrict__ scales,
                                                                  void* __restrict__ dst, size_t begin, size_t n, unsigned block_size, float scale)
{
    const size_t stride = (size_t)gridDim.x * kThreads;
    for (size_t i = begin + (size_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += stride)
    {
        const uint32_t byte = src[i >> 1];
        const uint32_t nib = (i & 1u) ? (byte >> 4) : (byte & 0xFu);
        const float s = BLOCKSCALE ? e4m3_to_f32(scales[i / block_size]) : scale;
        store_one<DST>(dst, i, fp4_to_f32(nib) * s);
    }
}

template <int DST, bool BLOCKSCALE>
int launch_dequant4(const void* src, const void* scales, void* dst, unsigned n, unsigned block_size, float scale, const char* what)
{
    if (n == 0) { return 0; }
    const bool aligned = (((uintptr_t)src & 7u) | ((uintptr_t)dst & 15u)) == 0;
    const bool vec_ok = aligned && (!BLOCKSCALE || block_size % 16 == 0);
    const size_t n_vec = vec_ok ? (size_t)n / 16 : 0;
    if (n_vec)
    {
        dequant4_vec_kernel<DST, BLOCKSCALE><<<grid_for(n_vec), kThreads, 0, stream()>>>((const uint8_t*)src, (const uint8_t*)scales, dst, n_vec, block_size, scale);
    }
    const size_t done = n_vec * 16;
    if (done < n)
    {
        dequant4_scalar_kernel<DST, BLOCKSCALE><<<grid_for(n - done), kThreads, 0, stream()>>>((const uint8_t*)src, (const uint8_t*)scales, dst, done, n, block_size, scale);
    }
    return finish(what);
}

// ---- the remaining pairs of the table: one element per lane, not on the hot path

// Truncating encoders of the reference (cccc-cuda/cuda_functions.cu:2382-2412, :2694-2724, :2796-2832)
__device__ __forceinline__ uint32_t f32_to_e5m2_trunc(float f)
{
    const uint32_t u = f32_to_bits(f);
    const uint32_t mag = u & 0x7FFFFFFFu;
    const uint32_t sign = (u >> 31) << 7;
    if (mag > 0x7F800000u) { return 0x7Cu; }
    if (mag == 0x7F800000u) { return sign | 0x7Cu; }
    const int fe = (int)((u >> 23) & 255u) - 127;
    const uint32_t fm = u & 0x7FFFFFu;
    if (fe > 15 || (fe == 15 && fm >= 0xE00000u)) { return sign | 0x7Bu; }
    const int e8 = fe + 15;
    if (e8 <= 0)
    {
        const int shift = 7 - fe;
        if (shift >= 32) { return sign; }
        return sign | (((fm | 0x800000u) >> shift) & 3u);
    }
    return sign | ((uint32_t)(e8 & 31) << 2) | (fm >> 21);
}

__device__ __forceinline__ uint32_t f32_to_e4m3_trunc(float f)
{
    const uint32_t u = f32_to_bits(f);
    const uint32_t sign = (u >> 31) << 7;
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) { return 0x7Fu; }
    const int fe = (int)((u >> 23) & 255u) - 127;
    const uint32_t fm = u & 0x7FFFFFu;
    if (fe > 8 || (fe == 8 && fm >= 0xC00000u)) { return sign | 0x7Eu; }
    const int e8 = fe + 7;
    if (e8 <= 0)
    {
        const int shift = 14 - fe;
        if (shift >= 32) { return sign; }
        return sign | (((fm | 0x800000u) >> shift) & 7u);
    }
    uint32_t m8 = fm >> 20;
    if (e8 == 15 && m8 == 7u) { m8 = 6u; }
    return sign | ((uint32_t)(e8 & 15) << 3) | m8;
}

__device__ __forceinline__ uint32_t f32_to_fp4(float f)
{
    const uint32_t s = (f < 0.0f) ? 8u : 0u;
    const float a = (f < 0.0f) ? -f : f;
    const uint32_t code = a < 0.25f ? 0u : a < 0.75f ? 1u : a < 1.25f ? 2u : a < 1.75f ? 3u : a < 2.5f ? 4u : a < 3.5f ? 5u : a < 5.0f ? 6u : 7u;
    return s | code;
}

__device__ __forceinline__ float load_plain(const void* src, int type, size_t i)
{
    if (type == DT_FLOAT) { return ((const float*)src)[i]; }
    if (type == DT_HALF) { return (float)((const _Float16*)src)[i]; }
    return bf16_bits_to_f32(((const uint16_t*)src)[i]);
}

// Plain casts (no scale): float->bf16, half->float, half->bf16, bf16->float, bf16->half.
// BF16 results round to nearest even; NaN inputs stay NaN (quiet bit forced).
__global__ __launch_bounds__(kThreads) void cast_kernel(const void* __restrict__ src, int src_type, void* __restrict__ dst, int dst_type, size_t n)
{
    const size_t stride = (size_t)gridDim.x * kThreads;
    for (size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += stride)
    {
        const float v = load_plain(src, src_type, i);
        if (dst_type == DT_FLOAT) { ((float*)dst)[i] = v; }
        else if (dst_type == DT_HALF) { ((uint16_t*)dst)[i] = (uint16_t)f32_to_half_bits(v); }
        else
        {
            const uint32_t bits = (v != v) ? ((f32_to_bits(v) >> 16) | 0x40u) : f32_to_bf16_bits(v);
            ((uint16_t*)dst)[i] = (uint16_t)bits;
        }
    }
}

// Quantising casts: float|bf16 -> e4m3, float -> e5m2 (value * scale, truncating encoders).
__global__ __launch_bounds__(kThreads) void encode8_kernel(const void* __restrict__ src, int src_type, uint8_t* __restrict__ dst, int dst_type, size_t n, float scale)
{
    const size_t stride = (size_t)gridDim.x * kThreads;
    for (size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += stride)
    {
        const float v = load_plain(src, src_type, i) * scale;
        dst[i] = (uint8_t)(dst_type == DT_E5M2 ? f32_to_e5m2_trunc(v) : f32_to_e4m3_trunc(v));
    }
}

// float -> packed FP4 with a per-tensor scale; one lane per output byte.
__global__ __launch_bounds__(kThreads) void encode4_kernel(const float* __restrict__ src, uint8_t* __restrict__ dst, size_t n, float scale)
{
    const size_t n_bytes = (n + 1) / 2;
    const size_t stride = (size_t)gridDim.x * kThreads;
    for (size_t b = (size_t)blockIdx.x * kThreads + threadIdx.x; b < n_bytes; b += stride)
    {
        const size_t e0 = 2 * b;
        const uint32_t lo = f32_to_fp4(src[e0] * scale);
        const uint32_t hi = (e0 + 1 < n) ? f32_to_fp4(src[e0 + 1] * scale) : 0u;
        dst[b] = (uint8_t)(lo | (hi << 4));
    }
}

// float -> FP4 nibbles + truncating E4M3 dequant scale per block; one lane per block.
__global__ __launch_bounds__(kThreads) void encode4_blockscale_kernel(const float* __restrict__ src, uint8_t* __restrict__ nibbles, uint8_t* __restrict__ scales,
                                                                     size_t n, unsigned block_size)
{
    const size_t n_blocks = (n + block_size - 1) / block_size;
    const size_t stride = (size_t)gridDim.x * kThreads;
    for (size_t b = (size_t)blockIdx.x * kThreads + threadIdx.x; b < n_blocks; b += stride)
    {
        const size_t lo = b * block_size;
        const size_t hi = (lo + block_size < n) ? lo + block_size : n;
        float amax = 0.0f;
        for (size_t i = lo; i < hi; i++) { amax = fmaxf(amax, fabsf(src[i])); }
        const float fwd = (amax > 1e-10f) ? (6.0f / amax) : 1.0f;
        const float dq = (amax > 1e-10f) ? (amax / 6.0f) : 1.0f;
        scales[b] = (uint8_t)f32_to_e4m3_trunc(dq);
        for (size_t i = lo; i < hi; i += 2)
        {
            const uint32_t l = f32_to_fp4(src[i] * fwd);
            const uint32_t h = (i + 1 < n) ? f32_to_fp4(src[i + 1] * fwd) : 0u;
            nibbles[i >> 1] = (uint8_t)(l | (h << 4));
        }
    }
}

// Largest magnitude.  16-byte loads over the aligned body (scalar loads for a misaligned pointer and the tail), wave
// reduction through lane reads, the four waves of a workgroup through LDS, then at most one atomic per workgroup on the
// bit pattern (non-negative floats order like unsigned integers) -- and none when the value already stored is at least as
// large: thousands of atomics on one address are served one after the other (190 us for 16 k of them, whatever n was).
// NaN inputs are skipped by fmaxf as before.
__global__ __launch_bounds__(kThreads) void absmax_kernel(const void* __restrict__ src, int src_type, size_t n, unsigned int* __restrict__ out)
{
    __shared__ float part[kThreads / 64];
    const size_t stride = (size_t)gridDim.x * kThreads;
    const size_t first = (size_t)blockIdx.x * kThreads + threadIdx.x;
    float m = 0.0f;
    const size_t per = src_type == DT_FLOAT ? 4 : 8;            // elements per 16-byte load
    const size_t n_vec = ((uintptr_t)src & 15u) == 0 ? n / per : 0;
    for (size_t c = first; c < n_vec; c += stride)
    {
        const u32x4 v = ((const u32x4*)src)[c];
#pragma unroll
        for (int d = 0; d < 4; d++)
        {
            if (src_type == DT_FLOAT) { m = fmaxf(m, fabsf(bits_to_f32(v[d]))); }
            else if (src_type == DT_HALF) { m = fmaxf(m, fmaxf(fabsf(half_bits_to_f32(v[d] & 0xFFFFu)), fabsf(half_bits_to_f32(v[d] >> 16)))); }
            else { m = fmaxf(m, fmaxf(fabsf(bf16_bits_to_f32(v[d] & 0xFFFFu)), fabsf(bf16_bits_to_f32(v[d] >> 16)))); }
        }
    }
    for (size_t i = n_vec * per + first; i < n; i += stride) { m = fmaxf(m, fabsf(load_plain(src, src_type, i))); }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) { m = fmaxf(m, __shfl_xor(m, off)); }
    if ((threadIdx.x & 63) == 0) { part[threadIdx.x >> 6] = m; }
    __syncthreads();
    if (threadIdx.x == 0)
    {
        for (int w = 1; w < kThreads / 64; w++) { m = fmaxf(m, part[w]); }
        const unsigned int bits = f32_to_bits(m);
        if (bits > __atomic_load_n(out, __ATOMIC_RELAXED)) { atomicMax(out, bits); }
    }
}

}    // namespace

int hip_absmax(const void* src, int src_type, unsigned int n, void* d_result)
{
    if (src_type != DT_FLOAT && src_type != DT_HALF && src_type != DT_BF16) { return -1; }
    if (!d_result) { return -1; }
    const hipError_t err = hipMemsetAsync(d_result, 0, sizeof(float), stream());
    if (err != hipSuccess)
    {
        fprintf(stderr, "absmax clear failed: %s\n", hipGetErrorString(err));
        return 1;
    }
    if (n) { absmax_kernel<<<grid_for(n), kThreads, 0, stream()>>>(src, src_type, n, (unsigned int*)d_result); }
    return finish("absmax");
}

int hip_convert(const void* src, int src_type, void* dst, int dst_type, unsigned int n, float scale)
{
    if (src_type == dst_type && scale == 1.0f)
    {
        if (n == 0) { return 0; }
        const hipError_t err = hipMemcpyAsync(dst, src, (size_t)n, hipMemcpyDeviceToDevice, stream());
        if (err != hipSuccess)
        {
            fprintf(stderr, "convert copy failed: %s\n", hipGetErrorString(err));
            return 1;
        }
        return finish("convert");
    }
    if ((unsigned)src_type >= 7u || (unsigned)dst_type >= 7u) { return -1; }
    const int pair = src_type * 8 + dst_type;
    switch (pair)
    {
    case DT_E5M2 * 8 + DT_BF16: return launch_dequant8<DT_E5M2, DT_BF16>(src, dst, n, scale, "fp8e5m2_to_bf16");
    case DT_E5M2 * 8 + DT_FLOAT: return launch_dequant8<DT_E5M2, DT_FLOAT>(src, dst, n, scale, "fp8e5m2_to_float");
    case DT_E5M2 * 8 + DT_HALF: return launch_dequant8<DT_E5M2, DT_HALF>(src, dst, n, scale, "fp8e5m2_to_half");
    case DT_E4M3 * 8 + DT_BF16: return launch_dequant8<DT_E4M3, DT_BF16>(src, dst, n, scale, "fp8e4m3_to_bf16");
    case DT_E4M3 * 8 + DT_FLOAT: return launch_dequant8<DT_E4M3, DT_FLOAT>(src, dst, n, scale, "fp8e4m3_to_float");
    case DT_E4M3 * 8 + DT_HALF: return launch_dequant8<DT_E4M3, DT_HALF>(src, dst, n, scale, "fp8e4m3_to_half");
    case DT_FP4 * 8 + DT_BF16: return launch_dequant4<DT_BF16, false>(src, nullptr, dst, n, 1, scale, "fp4_to_bf16");
    case DT_FP4 * 8 + DT_FLOAT: return launch_dequant4<DT_FLOAT, false>(src, nullptr, dst, n, 1, scale, "fp4_to_float");
    case DT_FLOAT * 8 + DT_BF16:
    case DT_HALF * 8 + DT_FLOAT:
    case DT_HALF * 8 + DT_BF16:
    case DT_BF16 * 8 + DT_FLOAT:
    case DT_BF16 * 8 + DT_HALF:
        if (n) { cast_kernel<<<grid_for(n), kThreads, 0, stream()>>>(src, src_type, dst, dst_type, n); }
        return finish("convert_cast");
    case DT_FLOAT * 8 + DT_E4M3:
    case DT_FLOAT * 8 + DT_E5M2:
    case DT_BF16 * 8 + DT_E4M3:
        if (n) { encode8_kernel<<<grid_for(n), kThreads, 0, stream()>>>(src, src_type, (uint8_t*)dst, dst_type, n, scale); }
        return finish("convert_to_fp8");
    case DT_FLOAT * 8 + DT_FP4:
        if (n) { encode4_kernel<<<grid_for((n + 1) / 2), kThreads, 0, stream()>>>((const float*)src, (uint8_t*)dst, n, scale); }
        return finish("float_to_fp4");
    default: return -1;
    }
}

int hip_fp4_blockscale_to_bf16(const void* src_nibbles, const void* src_scales, void* dst, unsigned int n_elems, unsigned int block_size)
{
    if (block_size == 0 || !src_scales) { return -1; }
    return launch_dequant4<DT_BF16, true>(src_nibbles, src_scales, dst, n_elems, block_size, 1.0f, "fp4_blockscale_to_bf16");
}

int hip_float_to_fp4_blockscale(const void* src, void* dst_nibbles, void* dst_scales, unsigned int n_elems, unsigned int block_size)
{
    if (block_size == 0 || (block_size & 1u)) { return -1; }
    if (n_elems == 0) { return 0; }
    const size_t n_blocks = ((size_t)n_elems + block_size - 1) / block_size;
    encode4_blockscale_kernel<<<grid_for(n_blocks), kThreads, 0, stream()>>>((const float*)src, (uint8_t*)dst_nibbles, (uint8_t*)dst_scales, n_elems, block_size);
    return finish("float_to_fp4_blockscale");
}
