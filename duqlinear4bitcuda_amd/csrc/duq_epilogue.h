// The fp16 dequant epilogues, one rounding per operator, shared by the stand-alone
// dequant kernels and the fused GEMM so that both give identical bits.
//   sym       : src/kernels/quant.cu:64-81      asym      : src/kernels/quant.cu:149-169
//   sym dual  : src/kernels/quant2.cu:62-83     asym dual : src/kernels/quant2.cu:158-186
// Mode 4 has no counterpart in the reference: operands hold signed-shifted codes c = u - 8 with
// shifted zero points z (x ~ s * (c - z)), and the epilogue applies the exact correction
//   corr = acc - z_row * (R_col - K * z_col) - z_col * R_row,   y = h(f32(corr) * (f32(s_row) * f32(s_col)))
// in 32-bit integers (R = per-row / per-column sums of the shifted codes; the column term is
// precomputed with the weights).
#pragma once
#include "duq_device.h"
#include "duq_launch.h"

namespace duq {

// Column-side parameters of one output column, resolved once per column:
// the dual modes pick between the two per-column sets here.
struct ColParams {
    f16 s;
    f16 z;
    f16 bias;
    int rs;  // mode 4
};

// Row-side parameters of one output row.
struct RowEpi {
    f16 s;
    f16 z;
    int rs;  // mode 4
};

// Batched launches (one problem per blockIdx.z / blockIdx.y, every tensor contiguous over the batch): move the
// per-row arrays by b * rows and the per-column ones by b * cols elements.
__device__ __forceinline__ void batch_shift(Epilogue &e, uint32_t b, uint32_t rows, uint32_t cols)
{
    const uint64_t r = (uint64_t)b * rows, c = (uint64_t)b * cols;
    if (e.s_row) e.s_row += r;
    if (e.z_row) e.z_row += r;
    if (e.rs_row) e.rs_row += r;
    if (e.s_col_1) e.s_col_1 += c;
    if (e.z_col_1) e.z_col_1 += c;
    if (e.s_col_2) e.s_col_2 += c;
    if (e.z_col_2) e.z_col_2 += c;
    if (e.bias) e.bias += c;
    if (e.rs_col) e.rs_col += c;
    if (e.rs_col_2) e.rs_col_2 += c;
}

template <int MODE>
__device__ __forceinline__ RowEpi load_row(const Epilogue &e, uint32_t row)
{
    RowEpi r;
    r.s = bits_to_f16(e.s_row[row]);
    r.z = (MODE == 1 || MODE == 3 || MODE == 4) ? bits_to_f16(e.z_row[row]) : (f16)0;
    r.rs = MODE == 4 ? e.rs_row[row] : 0;
    return r;
}

template <int MODE, bool BIAS>
__device__ __forceinline__ ColParams load_col(const uint16_t *s1, const uint16_t *z1, const uint16_t *s2,
                                              const uint16_t *z2, const uint16_t *bias, uint32_t col,
                                              const int32_t *rs = nullptr)
{
    ColParams c;
    c.z = (f16)0;
    c.bias = (f16)0;
    c.rs = 0;
    if (MODE == 0) {
        c.s = bits_to_f16(s1[col]);
    } else if (MODE == 4) {
        c.s = bits_to_f16(s1[col]);
        c.z = bits_to_f16(z1[col]);
        c.rs = rs[col];
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
__device__ __forceinline__ uint16_t dequant_one(int acc, const RowEpi &r, const ColParams &c)
{
    f16 y;
    if (MODE == 4) {
        // 32-bit wrapping integer arithmetic; zero points are integer-valued binary16 numbers
        const uint32_t zr = (uint32_t)rint_i32((float)r.z), zc = (uint32_t)rint_i32((float)c.z);
        const int corr = (int)((uint32_t)acc - zr * (uint32_t)c.rs - zc * (uint32_t)r.rs);
        const float ss = (float)r.s * (float)c.s;  // exact: 11-bit x 11-bit significands
        float prod = (float)corr * ss;
        asm volatile("" : "+v"(prod));  // round to float32 here, then to binary16 (no single-rounding mixed FMA)
        y = (f16)prod;
    } else {
        const f16 e = acc_to_f16(acc);
        const f16 ss = r.s * c.s;  // h(s_row * s_col)
        if (MODE == 0 || MODE == 2) {
            y = ss * e;
        } else {
            const f16 t = (e - r.z) - c.z;
            y = ss * t;
        }
    }
    if (BIAS) y = y + c.bias;
    return f16_to_bits(y);
}

// The same for an accumulator that arrives as an integer-valued float32 (|acc| < 2^24): the
// binary16 rounding of the float is the rounding of the integer, so only mode 4 converts back.
template <int MODE, bool BIAS>
__device__ __forceinline__ uint16_t dequant_one(float acc, const RowEpi &r, const ColParams &c)
{
    if (MODE == 4) return dequant_one<MODE, BIAS>((int)acc, r, c);
    const f16 e = (f16)acc;
    const f16 ss = r.s * c.s;
    f16 y;
    if (MODE == 0 || MODE == 2) {
        y = ss * e;
    } else {
        const f16 t = (e - r.z) - c.z;
        y = ss * t;
    }
    if (BIAS) y = y + c.bias;
    return f16_to_bits(y);
}

// Two neighbouring columns of one row at once, on the packed binary16 instructions (each lane of a
// packed operation rounds like the scalar one): the low half of the result is column c0.
template <int MODE, bool BIAS, typename ACC>
__device__ __forceinline__ uint32_t dequant_pair(ACC acc0, ACC acc1, const RowEpi &r, const ColParams &c0,
                                                 const ColParams &c1)
{
    if (MODE == 4)
        return (uint32_t)dequant_one<MODE, BIAS>(acc0, r, c0) | ((uint32_t)dequant_one<MODE, BIAS>(acc1, r, c1) << 16);
    const v2h e = v2h{(f16)(float)acc0, (f16)(float)acc1};  // int32 or integer-valued float32: one rounding
    const v2h ss = v2h{r.s, r.s} * v2h{c0.s, c1.s};
    v2h y;
    if (MODE == 0 || MODE == 2) {
        y = ss * e;
    } else {
        const v2h t = (e - v2h{r.z, r.z}) - v2h{c0.z, c1.z};
        y = ss * t;
    }
    if (BIAS) y = y + v2h{c0.bias, c1.bias};
    return __builtin_bit_cast(uint32_t, y);
}

// Row-sum epilogue of the dual-uniform layer for one output (definition: include/duq_hip.h,
// duq_asym_dual_rowsum_dequant_host), shared by the stand-alone kernel and the fused GEMM so that both give
// identical bits.  xlo / xhi and wlo / whi: the first eight bytes of the packed activation and weight rows, xhi
// masked to its two nibbles (input columns 8, 9); rxl = sum of the activation row's codes 0..9, rxr = of the others.
// I24: every factor of the four products is known to lie inside the signed 24-bit range (fits_i24), so they run
// on the full-rate 24-bit multiplier; the low 32 bits of those products are the wrapping 32-bit products.
__device__ __forceinline__ bool fits_i24(uint32_t v) { return (uint32_t)((int)v + (1 << 23)) < (1u << 24); }

template <bool I24 = false>
__device__ __forceinline__ uint16_t dual_rowsum_one(int acc, uint32_t xlo, uint32_t xhi, uint32_t zx, uint32_t rxl,
                                                    uint32_t rxr, float sx, uint32_t wlo, uint32_t whi, float s1, float s2,
                                                    uint32_t z1, uint32_t z2, uint32_t a1, uint32_t a2, bool with_bias,
                                                    f16 bias)
{
    const uint32_t accl = (uint32_t)__builtin_amdgcn_sdot8((int)xhi, (int)whi, __builtin_amdgcn_sdot8((int)xlo, (int)wlo, 0, false), false);
    // 32-bit wrapping integer arithmetic, like the single-range row-sum epilogue
    auto mul = [](uint32_t a, uint32_t b) -> uint32_t {
        return I24 ? (uint32_t)__mul24((int)a, (int)b) : a * b;
    };
    const int corr_l = (int)(accl - mul(zx, a1) - mul(z1, rxl));
    const int corr_r = (int)(((uint32_t)acc - accl) - mul(zx, a2) - mul(z2, rxr));
    float t1 = (float)corr_l * (sx * s1);  // sx * s: exact (11-bit significands)
    float t2 = (float)corr_r * (sx * s2);
    asm volatile("" : "+v"(t1), "+v"(t2));  // each product rounded to float32 on its own
    float t = t1 + t2;
    asm volatile("" : "+v"(t));             // the sum rounded to float32, then to binary16
    f16 y = (f16)t;
    if (with_bias) y = y + bias;
    return f16_to_bits(y);
}

// Row-side and column-side records of that epilogue for kernels that finish one output per thread (the decode
// kernels): everything dual_rowsum_one needs of one activation row / one weight row.
struct DualRow {
    uint32_t xlo, xhi;  // codes of input columns 0..7 / 8, 9 (xhi masked to its two nibbles)
    uint32_t zx, rxl, rxr;
    float sx;
};
struct DualCol {
    uint32_t wlo, whi;
    uint32_t z1, z2, a1, a2;
    float s1, s2;
    f16 bias;
};

// sum of the ten codes held in xlo (eight signed nibbles) and xhi (two)
__device__ __forceinline__ uint32_t dual_head_sum(uint32_t xlo, uint32_t xhi)
{
    return (uint32_t)__builtin_amdgcn_sdot8((int)xhi, 0x11111111, __builtin_amdgcn_sdot8((int)xlo, 0x11111111, 0, false), false);
}

// xq: the packed activation row (its first eight bytes are read), kbytes = K / 2
__device__ __forceinline__ DualRow load_dual_row(const Epilogue &e, const uint8_t *xq, uint32_t kbytes, uint32_t row)
{
    DualRow r;
    const v2u head = *reinterpret_cast<const v2u *>(xq + (uint64_t)row * kbytes);
    r.xlo = head[0];
    r.xhi = head[1] & 0xFFu;
    r.zx = (uint32_t)rint_i32((float)bits_to_f16(e.z_row[row]));
    r.sx = (float)bits_to_f16(e.s_row[row]);
    r.rxl = dual_head_sum(r.xlo, r.xhi);
    r.rxr = (uint32_t)e.rs_row[row] - r.rxl;
    return r;
}

__device__ __forceinline__ DualCol load_dual_col(const Epilogue &e, const uint8_t *w, uint32_t kbytes, uint32_t col, bool bias)
{
    DualCol c;
    const v2u head = *reinterpret_cast<const v2u *>(w + (uint64_t)col * kbytes);
    c.wlo = head[0];
    c.whi = head[1];
    c.s1 = (float)bits_to_f16(e.s_col_1[col]);
    c.s2 = (float)bits_to_f16(e.s_col_2[col]);
    c.z1 = (uint32_t)rint_i32((float)bits_to_f16(e.z_col_1[col]));
    c.z2 = (uint32_t)rint_i32((float)bits_to_f16(e.z_col_2[col]));
    c.a1 = (uint32_t)e.rs_col[col];
    c.a2 = (uint32_t)e.rs_col_2[col];
    c.bias = bias ? bits_to_f16(e.bias[col]) : (f16)0;
    return c;
}

__device__ __forceinline__ uint16_t dual_finish(int acc, const DualRow &r, const DualCol &c, bool bias)
{
    return dual_rowsum_one<false>(acc, r.xlo, r.xhi, r.zx, r.rxl, r.rxr, r.sx, c.wlo, c.whi, c.s1, c.s2, c.z1, c.z2, c.a1, c.a2,
                                  bias, c.bias);
}

// Column parameters of four consecutive output columns n0 .. n0+3, fetched with 64-bit
// loads when the arrays allow it (`vec`: 8-byte aligned bases and n0 + 3 < cols).
template <int MODE, bool BIAS>
struct QuadCols {
    ColParams c[4];
};

__device__ __forceinline__ void load4_f16(const uint16_t *ptr, uint32_t n0, uint32_t cols, bool vec, uint16_t (&out)[4])
{
    if (vec && n0 + 3 < cols) {
        const v2u v = *reinterpret_cast<const v2u *>(ptr + n0);
        out[0] = (uint16_t)(v[0] & 0xFFFFu);
        out[1] = (uint16_t)(v[0] >> 16);
        out[2] = (uint16_t)(v[1] & 0xFFFFu);
        out[3] = (uint16_t)(v[1] >> 16);
    } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) out[r] = ptr[min(n0 + r, cols - 1)];
    }
}

template <int MODE, bool BIAS>
__device__ __forceinline__ QuadCols<MODE, BIAS> load_quad_cols(const uint16_t *s1, const uint16_t *z1,
                                                               const uint16_t *s2, const uint16_t *z2,
                                                               const uint16_t *bias, uint32_t n0, uint32_t cols,
                                                               bool vec, const int32_t *rs = nullptr)
{
    QuadCols<MODE, BIAS> q;
    uint16_t a[4], b[4];
    load4_f16(s1, n0, cols, vec, a);
    if (MODE == 2 || MODE == 3) load4_f16(s2, n0, cols, vec, b);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t col = n0 + r;
        const bool first = MODE == 2 ? col < (uint32_t)kQuantColK : col == 0;  // see load_col
        q.c[r].s = bits_to_f16((MODE == 2 || MODE == 3) ? (first ? a[r] : b[r]) : a[r]);
        q.c[r].z = (f16)0;
        q.c[r].bias = (f16)0;
        q.c[r].rs = MODE == 4 ? rs[min(col, cols - 1)] : 0;
    }
    if (MODE == 1 || MODE == 3 || MODE == 4) {
        load4_f16(z1, n0, cols, vec, a);
        if (MODE == 3) load4_f16(z2, n0, cols, vec, b);
#pragma unroll
        for (int r = 0; r < 4; ++r) q.c[r].z = bits_to_f16(MODE == 3 ? ((n0 + r) == 0 ? a[r] : b[r]) : a[r]);
    }
    if (BIAS) {
        load4_f16(bias, n0, cols, vec, a);
#pragma unroll
        for (int r = 0; r < 4; ++r) q.c[r].bias = bits_to_f16(a[r]);
    }
    return q;
}

// Same selection as load_quad_cols, from raw 64-bit words fetched earlier (four binary16
// values per word, column n0 first).
template <int MODE, bool BIAS>
__device__ __forceinline__ QuadCols<MODE, BIAS> quad_cols_from_raw(v2u s1, v2u z1, v2u s2, v2u z2, v2u bias, uint32_t n0,
                                                                   v4i rs = v4i{0, 0, 0, 0})
{
    auto pick = [](v2u v, int r) -> uint16_t { return (uint16_t)((r & 1) ? (v[r >> 1] >> 16) : (v[r >> 1] & 0xFFFFu)); };
    QuadCols<MODE, BIAS> q;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t col = n0 + r;
        const bool first = MODE == 2 ? col < (uint32_t)kQuantColK : col == 0;
        q.c[r].s = bits_to_f16((MODE == 2 || MODE == 3) ? (first ? pick(s1, r) : pick(s2, r)) : pick(s1, r));
        q.c[r].rs = MODE == 4 ? rs[r] : 0;
        q.c[r].z = (MODE == 1 || MODE == 4) ? bits_to_f16(pick(z1, r))
                               : (MODE == 3 ? bits_to_f16(col == 0 ? pick(z1, r) : pick(z2, r)) : (f16)0);
        q.c[r].bias = BIAS ? bits_to_f16(pick(bias, r)) : (f16)0;
    }
    return q;
}

}  // namespace duq
