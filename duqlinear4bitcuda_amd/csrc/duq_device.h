// Device-side helpers shared by the gfx950 kernels: binary16 arithmetic with one
// rounding per operator, nibble packing, wavefront (64-lane) reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstddef>

#include <type_traits>

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

// ---- kernel arguments delivered in registers ------------------------------------------------------------
// gfx950 can hand a kernel the first 14 dwords of its arguments in scalar registers when the wavefront starts
// (compiled with -mllvm -amdgpu-kernarg-preload-count=14) instead of the kernel fetching them from the argument
// buffer with a scalar load, a fetch that a short kernel waits for with nothing to overlap it (measured: a kernel
// that only reads 8 MiB takes 2.66 us with its three arguments preloaded against 2.99 us).  Only leading scalar
// arguments qualify, not a parameter struct passed by value, so a kernel that wants this takes the first 56 bytes
// of its parameter struct once more as 14 dwords in front of the struct (DUQ_HEAD_DECL), and with_head() puts them
// back in place: fields of the first 56 bytes then come from registers, the others from the argument buffer.
// DUQ_LAUNCH_HEAD is the host side.  Pointers rebuilt this way have lost their address space: as_global() says
// again that one points to device memory (direct loads and stores through it would otherwise be flat ones).
#define DUQ_HEAD_DECL                                                                                                  \
    uint32_t h0, uint32_t h1, uint32_t h2, uint32_t h3, uint32_t h4, uint32_t h5, uint32_t h6, uint32_t h7, uint32_t h8, \
        uint32_t h9, uint32_t h10, uint32_t h11, uint32_t h12, uint32_t h13
#define DUQ_HEAD_USE h0, h1, h2, h3, h4, h5, h6, h7, h8, h9, h10, h11, h12, h13
constexpr int kHeadBytes = 56;

template <typename T>
__device__ __forceinline__ T with_head(const T &tail, DUQ_HEAD_DECL)
{
    static_assert(sizeof(T) >= kHeadBytes && std::is_trivially_copyable<T>::value, "parameter struct");
    T q = tail;
    const uint32_t hw[14] = {DUQ_HEAD_USE};
    __builtin_memcpy(&q, hw, kHeadBytes);
    return q;
}

template <typename T>
__device__ __forceinline__ __attribute__((address_space(1))) T *as_global(T *p)
{
    return (__attribute__((address_space(1))) T *)p;
}

// The same for a (wavefront-uniform) pointer variable or field, in place: uses that follow are resolved to device
// memory.  The empty asm keeps the compiler from folding the two casts away.
template <typename T>
__device__ __forceinline__ void to_global(T *&p)
{
    auto g = as_global(p);
    asm("" : "+s"(g));
    p = (T *)g;
}

#define DUQ_LAUNCH_HEAD(kernel, grid, block, lds, stream, params)                                                      \
    do {                                                                                                               \
        static_assert(sizeof(params) >= duq::kHeadBytes, "parameter struct");                                          \
        uint32_t duq_hw_[14];                                                                                          \
        __builtin_memcpy(duq_hw_, &(params), duq::kHeadBytes);                                                         \
        hipLaunchKernelGGL(kernel, grid, block, lds, stream, duq_hw_[0], duq_hw_[1], duq_hw_[2], duq_hw_[3], duq_hw_[4], \
                           duq_hw_[5], duq_hw_[6], duq_hw_[7], duq_hw_[8], duq_hw_[9], duq_hw_[10], duq_hw_[11],        \
                           duq_hw_[12], duq_hw_[13], params);                                                          \
    } while (0)

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

// 64-lane reductions, the same value in every lane: four DPP steps inside the rows of 16 lanes (two quad
// permutations, half-row mirror, row mirror: plain vector instructions, no trip through the LDS crossbar that a
// lane shuffle takes), then the four rows through scalar registers.
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_get(uint32_t v)
{
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}
template <typename T, typename OP>
__device__ __forceinline__ T wave_reduce_dpp(T v, OP op)
{
    auto step = [&](auto ctrl) {
        const uint32_t o = dpp_get<decltype(ctrl)::value>(__builtin_bit_cast(uint32_t, v));
        v = op(v, __builtin_bit_cast(T, o));
    };
    step(std::integral_constant<int, 0xB1>{});   // quad_perm [1,0,3,2]
    step(std::integral_constant<int, 0x4E>{});   // quad_perm [2,3,0,1]
    step(std::integral_constant<int, 0x141>{});  // row_half_mirror
    step(std::integral_constant<int, 0x140>{});  // row_mirror
    const uint32_t bits = __builtin_bit_cast(uint32_t, v);
    const T a = __builtin_bit_cast(T, (uint32_t)__builtin_amdgcn_readlane((int)bits, 0));
    const T b = __builtin_bit_cast(T, (uint32_t)__builtin_amdgcn_readlane((int)bits, 16));
    const T c = __builtin_bit_cast(T, (uint32_t)__builtin_amdgcn_readlane((int)bits, 32));
    const T d = __builtin_bit_cast(T, (uint32_t)__builtin_amdgcn_readlane((int)bits, 48));
    return op(op(a, b), op(c, d));
}
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v)
{
    return wave_reduce_dpp(v, [](uint32_t x, uint32_t y) { return max(x, y); });
}
__device__ __forceinline__ float wave_max_f32(float v)
{
    return wave_reduce_dpp(v, [](float x, float y) { return fmaxf(x, y); });
}
__device__ __forceinline__ float wave_min_f32(float v)
{
    return wave_reduce_dpp(v, [](float x, float y) { return fminf(x, y); });
}
__device__ __forceinline__ int wave_sum_i32(int v)
{
    return wave_reduce_dpp(v, [](int x, int y) { return x + y; });
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
