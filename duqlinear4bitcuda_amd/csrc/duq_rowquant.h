// Per-token scale (and zero point) and the 8-elements-to-one-word quantization step, shared by the
// stand-alone row quantizer (duq_quant.hip) and the decode kernels that quantize their activations
// themselves (duq_decode.hip), so that both give identical bits.
//   scale / zero : qlinear4bit/nn/quantizer.py:13, 27-31
//   codes        : src/kernels/quant.cu:11-45 (sym), 99-132 (asym)
#pragma once
#include "duq_device.h"

namespace duq {

// packed max of two |binary16| bit patterns per 32-bit word (NaN patterns win, as in torch.max)
__device__ __forceinline__ uint32_t pk_absmax_u16(uint32_t acc, uint32_t w)
{
    const v2us a = __builtin_bit_cast(v2us, acc);
    const v2us b = __builtin_bit_cast(v2us, w & 0x7FFF7FFFu);
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(a, b));
}

// 8 binary16 elements -> 8 codes in one word, element by element (every special case of the reference:
// NaN -> 0, saturation, wrapping add of the zero point)
template <bool ASYM>
__device__ __forceinline__ uint32_t quant8_exact(const v4u raw, float rcp, int qmax, int zi)
{
    uint32_t word = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const uint32_t w = raw[e >> 1];
        const f16 xv = bits_to_f16((uint16_t)((e & 1) ? (w >> 16) : (w & 0xFFFFu)));
        word |= (ASYM ? asym_code(xv, rcp, zi) : sym_code(xv, rcp, qmax)) << (4 * e);
    }
    return word;
}

// Statistics of one row -> scale, zero point and everything the quantization step needs.
template <bool ASYM>
struct RowQuant {
    f16 s, z;
    float rcp, rcp_fast;
    int zi, qmax;
    bool fast;
    v2h lo2, hi2;
    uint32_t zadd;

    // sym: amax_bits = largest |x| bit pattern of the row (above 0x7C00: a NaN).
    // asym: mn / mx = the row's minimum / maximum as float (NaN when the row holds one).
    __device__ __forceinline__ void init(uint32_t amax_bits, float mn_f, float mx_f, float clip, int qmax_)
    {
        z = (f16)0;
        if (!ASYM) {
            const f16 am = bits_to_f16((uint16_t)amax_bits);
            const f16 s0 = (f16)((float)am / 7.0f);
            // torch multiplies in float32, rounds to float32, then to binary16: keep the two
            // roundings apart (a mixed-precision FMA would round the exact product once).
            float sc = (float)s0 * clip;
            asm volatile("" : "+v"(sc));
            s = (f16)sc;
        } else {
            const f16 mn = (f16)mn_f, mx = (f16)mx_f;  // exact: both are binary16 values
            const f16 d = mx - mn;
            s = (f16)((float)d / 15.0f);
            const f16 neg = -mn;
            const f16 qz = (f16)((float)neg / (float)s);
            z = (f16)__builtin_rintf((float)qz);
        }
        setup(s, z, row_rcp(s), amax_bits, mn_f, mx_f, qmax_);
    }

    // The cheap part: scale, zero point and reciprocal already known (init computed them, here or in another
    // wavefront), derive the constants of the quantization step.
    __device__ __forceinline__ void setup(f16 s_, f16 z_, float rcp_, uint32_t amax_bits, float mn_f, float mx_f, int qmax_)
    {
        s = s_;
        z = z_;
        rcp = rcp_;
        qmax = qmax_;
        zi = ASYM ? rint_i32((float)z) : 0;
        // Rows whose statistics are finite (every realistic row) take the packed path: two
        // elements per instruction in binary16, rounding by adding 1536 (its ulp is 1, so the
        // sum is the nearest-even integer and its low byte is the code, sign-extended).  That path cannot
        // produce the NaN -> 0 conversions of the reference, which finite rows never need; any
        // row with a NaN / inf statistic, a zero scale on a non-zero row, or a zero point too
        // large for exact binary16 bounds runs the element-wise path.
        rcp_fast = rcp;
        const uint32_t s_bits = f16_to_bits(s) & 0x7FFFu;
        if (!ASYM) {
            const uint32_t am_bits = amax_bits & 0xFFFFu;
            fast = am_bits < 0x7C00u && s_bits < 0x7C00u && (s_bits != 0 || am_bits == 0);
            if (s_bits == 0) rcp_fast = 0.f;
        } else {
            fast = fabsf(mn_f) < 65520.f && fabsf(mx_f) < 65520.f && s_bits != 0 && s_bits < 0x7C00u && zi >= -480 &&
                   zi <= 480;
        }
        lo2 = ASYM ? v2h{(f16)(float)(-zi), (f16)(float)(-zi)} : v2h{(f16)-8.0f, (f16)-8.0f};
        hi2 = ASYM ? v2h{(f16)(float)(15 - zi), (f16)(float)(15 - zi)} : v2h{(f16)(float)qmax, (f16)(float)qmax};
        zadd = ASYM ? (((uint32_t)zi & 0xFFFFu) * 0x00010001u) : 0u;
    }

    // two binary16 values -> their codes in the low nibbles of bytes 0 and 2 (finite rows; the high nibbles of
    // those bytes hold the sign extension).  h(float(x) * rcp) for both halves is one mixed-precision
    // instruction each (binary16 source, float32 arithmetic, binary16 result).
    __device__ __forceinline__ uint32_t pair_bytes(uint32_t w) const
    {
        uint32_t d;
        asm("v_fma_mixlo_f16 %0, %1, %2, 0 op_sel_hi:[0,1,0]" : "=v"(d) : "v"(rcp_fast), "v"(w));
        asm("v_fma_mixhi_f16 %0, %1, %2, 0 op_sel:[0,1,0] op_sel_hi:[0,1,0]" : "+v"(d) : "v"(rcp_fast), "v"(w));
        v2h q = __builtin_bit_cast(v2h, d);
        q = __builtin_elementwise_min(__builtin_elementwise_max(q, lo2), hi2);
        q = q + v2h{(f16)1536.0f, (f16)1536.0f};
        uint32_t bits = __builtin_bit_cast(uint32_t, q);
        if (ASYM) {
            const v2us sum = __builtin_bit_cast(v2us, bits) + __builtin_bit_cast(v2us, zadd);
            bits = __builtin_bit_cast(uint32_t, sum);
        }
        return bits;
    }

    // 8 elements (one 128-bit load) -> one packed word, element 0 in the low nibble
    __device__ __forceinline__ uint32_t quant8(const v4u raw) const
    {
        if (!fast) return quant8_exact<ASYM>(raw, rcp, qmax, zi);
        const uint32_t b0 = pair_bytes(raw[0]), b1 = pair_bytes(raw[1]), b2 = pair_bytes(raw[2]), b3 = pair_bytes(raw[3]);
        // gather the code bytes (bytes 0 and 2 of every pair), then merge the low nibbles of neighbours into one byte
        const uint32_t p0 = __builtin_amdgcn_perm(b1, b0, 0x06040200u);
        const uint32_t p1 = __builtin_amdgcn_perm(b3, b2, 0x06040200u);
        const uint32_t t0 = (p0 & 0x0F0F0F0Fu) | ((p0 >> 4) & 0xF0F0F0F0u);
        const uint32_t t1 = (p1 & 0x0F0F0F0Fu) | ((p1 >> 4) & 0xF0F0F0F0u);
        return __builtin_amdgcn_perm(t1, t0, 0x06040200u);
    }
};

}  // namespace duq
