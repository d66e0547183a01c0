// The fp16 dequant epilogues, one rounding per operator, shared by the stand-alone
// dequant kernels and the fused GEMM so that both give identical bits.
//   sym       : src/kernels/quant.cu:64-81      asym      : src/kernels/quant.cu:149-169
//   sym dual  : src/kernels/quant2.cu:62-83     asym dual : src/kernels/quant2.cu:158-186
#pragma once
#include "duq_device.h"

namespace duq {

// Column-side parameters of one output column, resolved once per column:
// the dual modes pick between the two per-column sets here.
struct ColParams {
    f16 s;
    f16 z;
    f16 bias;
};

template <int MODE, bool BIAS>
__device__ __forceinline__ ColParams load_col(const uint16_t *s1, const uint16_t *z1, const uint16_t *s2,
                                              const uint16_t *z2, const uint16_t *bias, uint32_t col)
{
    ColParams c;
    c.z = (f16)0;
    c.bias = (f16)0;
    if (MODE == 0) {
        c.s = bits_to_f16(s1[col]);
    } else if (MODE == 1) {
        c.s = bits_to_f16(s1[col]);
        c.z = bits_to_f16(z1[col]);
    } else if (MODE == 2) {
        // col < QUANT_COL_K ? scale_col_1 : scale_col_2
        c.s = bits_to_f16(col < (uint32_t)kQuantColK ? s1[col] : s2[col]);
    } else {
        // the reference selector "(QUANT_COL_ST << col & 1)" is non-zero for column 0 only
        c.s = bits_to_f16(col == 0 ? s1[col] : s2[col]);
        c.z = bits_to_f16(col == 0 ? z1[col] : z2[col]);
    }
    if (BIAS) c.bias = bits_to_f16(bias[col]);
    return c;
}

template <int MODE, bool BIAS>
__device__ __forceinline__ uint16_t dequant_one(int acc, f16 s_row, f16 z_row, const ColParams &c)
{
    const f16 e = acc_to_f16(acc);
    const f16 ss = s_row * c.s;  // h(s_row * s_col)
    f16 y;
    if (MODE == 0 || MODE == 2) {
        y = ss * e;
    } else {
        const f16 t = (e - z_row) - c.z;
        y = ss * t;
    }
    if (BIAS) y = y + c.bias;
    return f16_to_bits(y);
}

}  // namespace duq
