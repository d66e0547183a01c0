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

// Running maximum and minimum of binary16 values, two per register, on the three-operand packed instructions of
// gfx950: two words (four elements) per instruction and statistic, where masking the sign and an unsigned
// maximum cost two instructions per word.  v_pk_maximum3_f16 / v_pk_minimum3_f16 return a NaN when an operand is
// one, so a row that holds a NaN ends with NaN statistics, as torch.max / torch.min do.
struct PkMinMax {
    uint32_t mx = 0xFC00FC00u;  // -inf, -inf
    uint32_t mn = 0x7C007C00u;  // +inf, +inf

    __device__ __forceinline__ void add2(uint32_t w0, uint32_t w1)
    {
        asm("v_pk_maximum3_f16 %0, %0, %1, %2" : "+v"(mx) : "v"(w0), "v"(w1));
        asm("v_pk_minimum3_f16 %0, %0, %1, %2" : "+v"(mn) : "v"(w0), "v"(w1));
    }
    __device__ __forceinline__ void add8(const v4u g)
    {
        add2(g[0], g[1]);
        add2(g[2], g[3]);
    }
    // both statistics over the 64 lanes (the same words in every lane)
    __device__ __forceinline__ void wave_reduce()
    {
        mx = wave_reduce_dpp(mx, [](uint32_t a, uint32_t b) {
            asm("v_pk_maximum3_f16 %0, %0, %1, %1" : "+v"(a) : "v"(b));
            return a;
        });
        mn = wave_reduce_dpp(mn, [](uint32_t a, uint32_t b) {
            asm("v_pk_minimum3_f16 %0, %0, %1, %1" : "+v"(a) : "v"(b));
            return a;
        });
    }
    // largest |x| bit pattern of the elements seen so far (above 0x7C00: a NaN; 0 when there were none)
    __device__ __forceinline__ uint32_t absmax_bits() const
    {
        if (mx == 0xFC00FC00u && mn == 0x7C007C00u) return 0u;  // only the empty state has max < min
        const uint32_t c = pk_absmax_u16(mx & 0x7FFF7FFFu, mn);
        return max(c & 0xFFFFu, c >> 16);
    }
    // minimum and maximum as float (NaNs dropped here: callers test absmax_bits() for them)
    __device__ __forceinline__ float min_f32() const
    {
        return fminf((float)bits_to_f16((uint16_t)(mn & 0xFFFFu)), (float)bits_to_f16((uint16_t)(mn >> 16)));
    }
    __device__ __forceinline__ float max_f32() const
    {
        return fmaxf((float)bits_to_f16((uint16_t)(mx & 0xFFFFu)), (float)bits_to_f16((uint16_t)(mx >> 16)));
    }
};

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
    bool fast, clamp_lo, clamp_hi;
    v2h lo2, hi2;
    uint32_t zadd;

    // sym: amax_bits = largest |x| bit pattern of the row (above 0x7C00: a NaN).
    // asym: mn / mx = the row's minimum / maximum as float (NaN when the row holds one).
    // The divisions by 7 and by 15 are multiplications by the rounded reciprocals: for every binary16 numerator
    // both give the same binary16 result (checked over all of them), and the zero point's quotient goes through
    // the same reciprocal as the codes (see row_rcp).
    __device__ __forceinline__ void init(uint32_t amax_bits, float mn_f, float mx_f, float clip, int qmax_)
    {
        z = (f16)0;
        float r;
        if (!ASYM) {
            const f16 am = bits_to_f16((uint16_t)amax_bits);
            float q7 = (float)am * (1.0f / 7.0f);
            asm volatile("" : "+v"(q7));
            const f16 s0 = (f16)q7;
            // torch multiplies in float32, rounds to float32, then to binary16: keep the two
            // roundings apart (a mixed-precision FMA would round the exact product once).
            float sc = (float)s0 * clip;
            asm volatile("" : "+v"(sc));
            s = (f16)sc;
            r = row_rcp(s);
        } else {
            const f16 mn = (f16)mn_f, mx = (f16)mx_f;  // exact: both are binary16 values
            const f16 d = mx - mn;
            float q15 = (float)d * (1.0f / 15.0f);
            asm volatile("" : "+v"(q15));
            s = (f16)q15;
            r = row_rcp(s);
            const f16 neg = -mn;
            float qzf = (float)neg * r;
            asm volatile("" : "+v"(qzf));
            const f16 qz = (f16)qzf;
            z = (f16)__builtin_rintf((float)qz);
        }
        setup(s, z, r, amax_bits, mn_f, mx_f, qmax_);
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
        //
        // h(x * rcp) grows with x, so the row's extreme values bound every quotient of the row, and a row whose
        // bound already rounds into the code range needs no clamp on that side.
        //   sym : |x| <= am, so every quotient lies in [-t, t] with t = h(am * rcp); no lower clamp when
        //         t <= 8.5 (ties go to the even integer), no upper one when t < qmax + 0.5.
        //   asym: the zero point is -rint(h(mn * rcp)) (rounding is symmetric), so the smallest code of the row
        //         is exactly 0 and the lower clamp never acts on a finite row; the upper one does not when
        //         rint(h(mx * rcp)) + zi <= 15.
        rcp_fast = rcp;
        const uint32_t s_bits = f16_to_bits(s) & 0x7FFFu;
        if (!ASYM) {
            const uint32_t am_bits = amax_bits & 0xFFFFu;
            fast = am_bits < 0x7C00u && s_bits < 0x7C00u && (s_bits != 0 || am_bits == 0);
            if (s_bits == 0) rcp_fast = 0.f;
            float tf = (float)bits_to_f16((uint16_t)am_bits) * rcp_fast;
            asm volatile("" : "+v"(tf));
            const float t = (float)(f16)tf;
            clamp_lo = !(t <= 8.5f);
            clamp_hi = !(t < (float)qmax + 0.5f);
        } else {
            fast = fabsf(mn_f) < 65520.f && fabsf(mx_f) < 65520.f && s_bits != 0 && s_bits < 0x7C00u && zi >= -480 &&
                   zi <= 480;
            float tf = mx_f * rcp_fast;
            asm volatile("" : "+v"(tf));
            const float t = __builtin_rintf((float)(f16)tf);
            clamp_lo = false;
            clamp_hi = !(t + (float)zi <= 15.f);
        }
        // every lane of a wavefront holds the same row statistics: tell the compiler, so that the choice of
        // path is a scalar branch
        fast = __builtin_amdgcn_readfirstlane((int)fast) != 0;
        clamp_lo = __builtin_amdgcn_readfirstlane((int)clamp_lo) != 0;
        clamp_hi = __builtin_amdgcn_readfirstlane((int)clamp_hi) != 0;
        lo2 = ASYM ? v2h{(f16)(float)(-zi), (f16)(float)(-zi)} : v2h{(f16)-8.0f, (f16)-8.0f};
        hi2 = ASYM ? v2h{(f16)(float)(15 - zi), (f16)(float)(15 - zi)} : v2h{(f16)(float)qmax, (f16)(float)qmax};
        zadd = ASYM ? (((uint32_t)zi & 0xFFFFu) * 0x00010001u) : 0u;
    }

    // 8 elements -> one packed word on the packed path (finite rows).  Per pair of binary16 values:
    // h(float(x) * rcp) for both halves is one mixed-precision instruction each (binary16 source, float32
    // arithmetic, binary16 result); clamp; add 1536, which leaves the codes in the low nibbles of bytes 0 and 2
    // (the high nibbles of those bytes hold the sign extension); asym adds the zero point.  The four pairs go
    // through each stage together so that no instruction waits for the one before it.
    template <bool LO, bool HI>
    __device__ __forceinline__ uint32_t quant8_packed(const v4u raw) const
    {
        uint32_t d[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
            asm("v_fma_mixlo_f16 %0, %1, %2, 0 op_sel_hi:[0,1,0]" : "=v"(d[i]) : "v"(rcp_fast), "v"(raw[i]));
#pragma unroll
        for (int i = 0; i < 4; ++i)
            asm("v_fma_mixhi_f16 %0, %1, %2, 0 op_sel:[0,1,0] op_sel_hi:[0,1,0]" : "+v"(d[i]) : "v"(rcp_fast), "v"(raw[i]));
        // written out: the generic minimum / maximum would first canonicalize the opaque results above, one
        // more instruction per pair that a finite row has no use for
        if (LO)
#pragma unroll
            for (int i = 0; i < 4; ++i) asm("v_pk_max_f16 %0, %0, %1" : "+v"(d[i]) : "v"(lo2));
        if (HI)
#pragma unroll
            for (int i = 0; i < 4; ++i) asm("v_pk_min_f16 %0, %0, %1" : "+v"(d[i]) : "v"(hi2));
        uint32_t b[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const v2h q = __builtin_bit_cast(v2h, d[i]) + v2h{(f16)1536.0f, (f16)1536.0f};
            b[i] = __builtin_bit_cast(uint32_t, q);
            if (ASYM) {
                const v2us sum = __builtin_bit_cast(v2us, b[i]) + __builtin_bit_cast(v2us, zadd);
                b[i] = __builtin_bit_cast(uint32_t, sum);
            }
        }
        // gather the code bytes (bytes 0 and 2 of every pair), then merge the low nibbles of neighbours into one
        // byte (a bit-field insert: low nibbles from p, high nibbles from p >> 4)
        const uint32_t p0 = __builtin_amdgcn_perm(b[1], b[0], 0x06040200u);
        const uint32_t p1 = __builtin_amdgcn_perm(b[3], b[2], 0x06040200u);
        uint32_t t0, t1;
        const uint32_t low = 0x0F0F0F0Fu;
        asm("v_bfi_b32 %0, %1, %2, %3" : "=v"(t0) : "s"(low), "v"(p0), "v"(p0 >> 4));
        asm("v_bfi_b32 %0, %1, %2, %3" : "=v"(t1) : "s"(low), "v"(p1), "v"(p1 >> 4));
        return __builtin_amdgcn_perm(t1, t0, 0x06040200u);
    }

    // 8 elements (one 128-bit load) -> one packed word, element 0 in the low nibble
    __device__ __forceinline__ uint32_t quant8(const v4u raw) const
    {
        if (!fast) return quant8_exact<ASYM>(raw, rcp, qmax, zi);
        if (!ASYM && clamp_lo) return quant8_packed<true, true>(raw);
        return clamp_hi ? quant8_packed<false, true>(raw) : quant8_packed<false, false>(raw);
    }

    // N units at once: the path is chosen once, so that the N independent chains of a path sit in one block of
    // straight-line code and the scheduler can interleave them (a unit's chain is eight instructions deep).  Units
    // a caller does not store may hold anything (zeros from loads past the row end): every path is total.
    template <int N>
    __device__ __forceinline__ void quant_units(const v4u (&raw)[N], uint32_t (&out)[N]) const
    {
        if (!fast) {
#pragma unroll
            for (int j = 0; j < N; ++j) out[j] = quant8_exact<ASYM>(raw[j], rcp, qmax, zi);
        } else if (!ASYM && clamp_lo) {
#pragma unroll
            for (int j = 0; j < N; ++j) out[j] = quant8_packed<true, true>(raw[j]);
        } else if (clamp_hi) {
#pragma unroll
            for (int j = 0; j < N; ++j) out[j] = quant8_packed<false, true>(raw[j]);
        } else {
#pragma unroll
            for (int j = 0; j < N; ++j) out[j] = quant8_packed<false, false>(raw[j]);
        }
    }
};

}  // namespace duq
