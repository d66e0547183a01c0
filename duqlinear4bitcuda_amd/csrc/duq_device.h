// Device-side helpers shared by the gfx950 kernels: binary16 arithmetic with one
// rounding per operator, nibble packing, wavefront (64-lane) reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace duq {

typedef _Float16 f16;
typedef int v4i __attribute__((ext_vector_type(4)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));
typedef unsigned short v2us __attribute__((ext_vector_type(2)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;
constexpr int kQuantColK = 10;  // include/quant.h:5 of the reference

__device__ __forceinline__ f16 bits_to_f16(uint16_t b) { return __builtin_bit_cast(f16, b); }
__device__ __forceinline__ uint16_t f16_to_bits(f16 v) { return __builtin_bit_cast(uint16_t, v); }

// float -> int32 with the hardware rule: truncation, saturation, NaN -> 0.  A C cast is
// undefined for NaN / out-of-range values, the instruction is not.
__device__ __forceinline__ int cvt_i32_sat(float v)
{
    int r;
    asm("v_cvt_i32_f32 %0, %1" : "=v"(r) : "v"(v));
    return r;
}

// nearest-even float -> int32, saturating, NaN -> 0 (the __half2int_rn rule once the
// operand is a widened binary16).
__device__ __forceinline__ int rint_i32(float v) { return cvt_i32_sat(__builtin_rintf(v)); }

// int32 accumulator -> binary16 with one rounding (|acc| < 2^24 is exact in float32;
// anything larger is far above 65520 and becomes +-inf either way).
__device__ __forceinline__ f16 acc_to_f16(int acc) { return (f16)(float)acc; }

__device__ __forceinline__ int clampi(int v, int lo, int hi) { return min(max(v, lo), hi); }

// 64-lane butterfly reductions (wavefront shuffles, no LDS traffic, no barrier).
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = max(v, (uint32_t)__shfl_xor((int)v, off, kWave));
    return v;
}
__device__ __forceinline__ float wave_max_f32(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}
__device__ __forceinline__ float wave_min_f32(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fminf(v, __shfl_xor(v, off, kWave));
    return v;
}

// Reciprocal used for x / s with x, s binary16: float32(x) * rcp is within two float32
// ulps of the true quotient, and no quotient of two binary16 numbers lies that close to
// a binary16 rounding boundary, so h(float32(x) * rcp) == h(x / s) for every pair.  The
// special cases follow the division too: s = 0 gives +-inf for x != 0 and NaN for x = 0.
__device__ __forceinline__ float row_rcp(f16 s) { return 1.0f / (float)s; }

// clamp(rint(h(x/s)), -8, qmax) as a two's-complement nibble
__device__ __forceinline__ uint32_t sym_code(f16 x, float rcp, int qmax)
{
    f16 hq = (f16)((float)x * rcp);
    int qi = clampi(rint_i32((float)hq), -8, qmax);
    return (uint32_t)qi & 0xFu;
}

// clamp(rint(h(x/s)) + zi, 0, 15); the add wraps like the 32-bit add of the reference
__device__ __forceinline__ uint32_t asym_code(f16 x, float rcp, int zi)
{
    f16 hq = (f16)((float)x * rcp);
    int qi = rint_i32((float)hq);
    int sum = (int)((uint32_t)qi + (uint32_t)zi);
    return (uint32_t)clampi(sum, 0, 15);
}

// clamp(rint(h(h(x/s) + z)), 0, 15)  (zero added in binary16 before the rounding)
__device__ __forceinline__ uint32_t asym_pre_code(f16 x, float rcp, f16 z)
{
    f16 hq = (f16)((float)x * rcp);
    f16 t = hq + z;
    return (uint32_t)clampi(rint_i32((float)t), 0, 15);
}

}  // namespace duq
