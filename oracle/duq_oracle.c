/*
 * Plain-C CPU oracle for the Linear4bit forward path.
 *
 * TEST INFRASTRUCTURE ONLY: a scalar restatement of the reference algorithm, used by
 * the tests, the smoke entry and the benchmark's cpu_baseline leg as the checker /
 * baseline.  The product library never links or loads it.
 *
 * It is written independently of the NumPy oracle (own binary16 conversion code, own
 * loops) so that the two can be checked against each other; each function cites the
 * reference lines it follows (paths relative to the reference checkout).
 *
 * Build: make -C oracle   ->  oracle/libduq_oracle.so
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define QUANT_COL_K 10 /* include/quant.h:5 */

/* ---------------- binary16 <-> binary32, bit level ---------------- */

static inline float u32_as_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_as_u32(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

float duqo_h2f(uint16_t hbits)
{
    uint32_t sign = (uint32_t)(hbits & 0x8000u) << 16;
    uint32_t exp = (hbits >> 10) & 0x1Fu;
    uint32_t man = hbits & 0x3FFu;
    if (exp == 0) {
        if (man == 0) return u32_as_f32(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * 5.9604644775390625e-08f;
        return sign ? -v : v;
    }
    if (exp == 31) return u32_as_f32(sign | 0x7F800000u | (man << 13));
    return u32_as_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* round-to-nearest-even float32 -> binary16 */
uint16_t duqo_f2h(float f)
{
    uint32_t u = f32_as_u32(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7FFFFFFFu;
    if (a >= 0x7F800000u) { /* inf / nan */
        if (a == 0x7F800000u) return sign | 0x7C00u;
        return sign | 0x7E00u | (uint16_t)((a >> 13) & 0x3FFu);
    }
    if (a >= 0x477FF000u) return sign | 0x7C00u;       /* >= 65520 -> inf */
    if (a < 0x33000001u) return sign;                   /* <= 2^-25 -> 0 (tie to even) */
    int32_t e = (int32_t)(a >> 23) - 127;
    uint32_t m = (a & 0x7FFFFFu) | 0x800000u;           /* 24-bit significand */
    int shift;                                           /* bits to drop */
    uint32_t base;
    if (e < -14) { shift = 13 + (-14 - e); base = 0; }   /* subnormal result */
    else { shift = 13; base = (uint32_t)(e + 15) << 10; m &= 0x7FFFFFu; }
    uint32_t keep = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    uint32_t r = base + keep;                            /* carry into exponent is right */
    if (rem > half || (rem == half && (keep & 1u))) r += 1u;
    return sign | (uint16_t)r;
}

static inline uint16_t hmul(uint16_t a, uint16_t b) { return duqo_f2h(duqo_h2f(a) * duqo_h2f(b)); }
static inline uint16_t hsub(uint16_t a, uint16_t b) { return duqo_f2h(duqo_h2f(a) - duqo_h2f(b)); }
static inline uint16_t hadd(uint16_t a, uint16_t b) { return duqo_f2h(duqo_h2f(a) + duqo_h2f(b)); }
static inline uint16_t hdiv(uint16_t a, uint16_t b) { return duqo_f2h(duqo_h2f(a) / duqo_h2f(b)); }

/* __int2half_rn (src/kernels/quant.cu:4-8): single rounding.  Going through double is
 * exact for any int32, and double -> binary16 below rounds once. */
static uint16_t int_to_half(int32_t v)
{
    double d = (double)v;
    double ad = fabs(d);
    if (ad < 16777216.0) return duqo_f2h((float)d);      /* exact in float32 */
    return (uint16_t)((v < 0 ? 0x8000u : 0u) | 0x7C00u); /* >= 65520 anyway */
}

/* __half2int_rn: nearest-even, saturating, NaN -> 0 */
static int32_t half_to_int_rn(uint16_t hbits)
{
    float f = duqo_h2f(hbits);
    if (f != f) return 0;
    if (f >= 2147483648.0f) return INT32_MAX;
    if (f <= -2147483648.0f) return INT32_MIN;
    return (int32_t)nearbyintf(f); /* default rounding mode: to nearest even */
}

static inline int32_t clampi(int32_t v, int32_t lo, int32_t hi) { return v < lo ? lo : (v > hi ? hi : v); }
static inline int32_t s4(uint32_t nib) { return (int32_t)((nib & 0xFu) ^ 8u) - 8; }

/* ---------------- A1 / A3: per-token scales ---------------- */

/* qlinear4bit/nn/quantizer.py:13 */
void duqo_sym_scales(const uint16_t *x, uint32_t rows, uint32_t cols, float clip, uint16_t *scale)
{
    for (uint32_t r = 0; r < rows; ++r) {
        float amax = 0.0f;
        int nan = 0;
        for (uint32_t c = 0; c < cols; ++c) {
            float v = fabsf(duqo_h2f(x[(size_t)r * cols + c]));
            if (v != v) nan = 1;
            if (v > amax) amax = v;
        }
        if (nan) amax = NAN;
        uint16_t s = duqo_f2h(amax / 7.0f);
        scale[r] = duqo_f2h(duqo_h2f(s) * clip);
    }
}

/* qlinear4bit/nn/quantizer.py:27-31 */
void duqo_asym_scales_zeros(const uint16_t *x, uint32_t rows, uint32_t cols, uint16_t *scale, uint16_t *zero)
{
    for (uint32_t r = 0; r < rows; ++r) {
        float mn = INFINITY, mx = -INFINITY;
        for (uint32_t c = 0; c < cols; ++c) {
            float v = duqo_h2f(x[(size_t)r * cols + c]);
            if (v < mn) mn = v;
            if (v > mx) mx = v;
        }
        uint16_t d = duqo_f2h(mx - mn);
        uint16_t s = duqo_f2h(duqo_h2f(d) / 15.0f);
        uint16_t neg = duqo_f2h(-mn);
        uint16_t qz = hdiv(neg, s);
        scale[r] = s;
        zero[r] = duqo_f2h(nearbyintf(duqo_h2f(qz)));
    }
}

/* ---------------- A2 / A3: quantize + pack ---------------- */

/* src/kernels/quant.cu:11-45; qmax = 6 on the device (include/common.h:53-54) */
void duqo_sym_quant(const uint16_t *x, const uint16_t *scale, uint32_t rows, uint32_t colsSrc,
                    uint32_t colsDst, int32_t qmax, uint8_t *q)
{
    for (uint32_t r = 0; r < rows; ++r)
        for (uint32_t cd = 0; cd < colsDst; ++cd) {
            uint8_t byte = 0;
            for (uint32_t i = 0; i < 2; ++i) {
                uint32_t c = cd * 2 + i;
                if (c >= colsSrc) continue;
                int32_t v = clampi(half_to_int_rn(hdiv(x[(size_t)r * colsSrc + c], scale[r])), -8, qmax);
                byte |= (uint8_t)((v & 0xF) << (4 * i));
            }
            q[(size_t)r * colsDst + cd] = byte;
        }
}

/* src/kernels/quant2.cu:9-45 */
void duqo_sym_dual_quant(const uint16_t *x, const uint16_t *scale_1, const uint16_t *scale_2, uint32_t rows,
                         uint32_t colsSrc, uint32_t colsDst, int32_t qmax, uint8_t *q)
{
    for (uint32_t r = 0; r < rows; ++r)
        for (uint32_t cd = 0; cd < colsDst; ++cd) {
            uint8_t byte = 0;
            for (uint32_t i = 0; i < 2; ++i) {
                uint32_t c = cd * 2 + i;
                if (c >= colsSrc) continue;
                uint16_t s = c < QUANT_COL_K ? scale_1[r] : scale_2[r];
                int32_t v = clampi(half_to_int_rn(hdiv(x[(size_t)r * colsSrc + c], s)), -8, qmax);
                byte |= (uint8_t)((v & 0xF) << (4 * i));
            }
            q[(size_t)r * colsDst + cd] = byte;
        }
}

/* src/kernels/quant.cu:99-132 */
void duqo_asym_quant(const uint16_t *x, const uint16_t *scale, const uint16_t *zeros, uint32_t rows,
                     uint32_t colsSrc, uint32_t colsDst, uint8_t *q)
{
    for (uint32_t r = 0; r < rows; ++r) {
        int32_t zi = half_to_int_rn(zeros[r]);
        for (uint32_t cd = 0; cd < colsDst; ++cd) {
            uint8_t byte = 0;
            for (uint32_t i = 0; i < 2; ++i) {
                uint32_t c = cd * 2 + i;
                if (c >= colsSrc) continue;
                int32_t qi = half_to_int_rn(hdiv(x[(size_t)r * colsSrc + c], scale[r]));
                int32_t sum = (int32_t)((uint32_t)qi + (uint32_t)zi); /* wraps like the device add */
                byte |= (uint8_t)((clampi(sum, 0, 15) & 0xF) << (4 * i));
            }
            q[(size_t)r * colsDst + cd] = byte;
        }
    }
}

/* src/kernels/quant2.cu:101-139 (zero added in binary16 before rounding) */
void duqo_asym_dual_quant(const uint16_t *x, const uint16_t *scale_1, const uint16_t *zeros_1,
                          const uint16_t *scale_2, const uint16_t *zeros_2, uint32_t rows, uint32_t colsSrc,
                          uint32_t colsDst, uint8_t *q)
{
    for (uint32_t r = 0; r < rows; ++r)
        for (uint32_t cd = 0; cd < colsDst; ++cd) {
            uint8_t byte = 0;
            for (uint32_t i = 0; i < 2; ++i) {
                uint32_t c = cd * 2 + i;
                if (c >= colsSrc) continue;
                uint16_t s = c < QUANT_COL_K ? scale_1[r] : scale_2[r];
                uint16_t z = c < QUANT_COL_K ? zeros_1[r] : zeros_2[r];
                uint16_t d = hadd(hdiv(x[(size_t)r * colsSrc + c], s), z);
                byte |= (uint8_t)((clampi(half_to_int_rn(d), 0, 15) & 0xF) << (4 * i));
            }
            q[(size_t)r * colsDst + cd] = byte;
        }
}

/* ---------------- A4: s4 x s4 -> s32 GEMM (src/kernels/gemm.cu:8-43) ---------------- */

void duqo_matmul_s4(const uint8_t *A, const uint8_t *B, uint32_t M, uint32_t N, uint32_t K, int32_t *C)
{
    const size_t kb = K / 2;
    int8_t *ua = (int8_t *)malloc((size_t)M * K + 1);
    int8_t *ub = (int8_t *)malloc((size_t)N * K + 1);
    for (size_t i = 0; i < (size_t)M * kb; ++i) {
        ua[2 * i] = (int8_t)s4(A[i]);
        ua[2 * i + 1] = (int8_t)s4(A[i] >> 4);
    }
    for (size_t i = 0; i < (size_t)N * kb; ++i) {
        ub[2 * i] = (int8_t)s4(B[i]);
        ub[2 * i + 1] = (int8_t)s4(B[i] >> 4);
    }
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < (int64_t)M; ++m) {
        const int8_t *ar = ua + (size_t)m * K;
        for (uint32_t n = 0; n < N; ++n) {
            const int8_t *br = ub + (size_t)n * K;
            int32_t acc = 0;
            for (uint32_t k = 0; k < K; ++k) acc += (int32_t)ar[k] * (int32_t)br[k];
            C[(size_t)m * N + n] = acc;
        }
    }
    free(ua);
    free(ub);
}

/* ---------------- A5 / A6 / A7: dequant epilogues ---------------- */

/* src/kernels/quant.cu:64-81 */
void duqo_sym_dequant(const int32_t *q, const uint16_t *scale_row, const uint16_t *scale_col, uint32_t rows,
                      uint32_t cols, uint16_t *x)
{
    for (uint32_t r = 0; r < rows; ++r)
        for (uint32_t c = 0; c < cols; ++c)
            x[(size_t)r * cols + c] = hmul(hmul(scale_row[r], scale_col[c]), int_to_half(q[(size_t)r * cols + c]));
}

/* src/kernels/quant2.cu:62-83 */
void duqo_sym_dual_dequant(const int32_t *q, const uint16_t *scale_row, const uint16_t *scale_col_1,
                           const uint16_t *scale_col_2, uint32_t rows, uint32_t cols, uint16_t *x)
{
    for (uint32_t r = 0; r < rows; ++r)
        for (uint32_t c = 0; c < cols; ++c) {
            uint16_t sc = c < QUANT_COL_K ? scale_col_1[c] : scale_col_2[c];
            x[(size_t)r * cols + c] = hmul(hmul(scale_row[r], sc), int_to_half(q[(size_t)r * cols + c]));
        }
}

/* src/kernels/quant.cu:149-169 */
void duqo_asym_dequant(const int32_t *q, const uint16_t *scale_row, const uint16_t *zeros_row,
                       const uint16_t *scale_col, const uint16_t *zeros_col, uint32_t rows, uint32_t cols,
                       uint16_t *x)
{
    for (uint32_t r = 0; r < rows; ++r)
        for (uint32_t c = 0; c < cols; ++c) {
            uint16_t e = int_to_half(q[(size_t)r * cols + c]);
            uint16_t inner = hsub(hsub(e, zeros_row[r]), zeros_col[c]);
            x[(size_t)r * cols + c] = hmul(hmul(scale_row[r], scale_col[c]), inner);
        }
}

/* src/kernels/quant2.cu:158-186: the selector is non-zero for column 0 only */
void duqo_asym_dual_dequant(const int32_t *q, const uint16_t *scale_row, const uint16_t *zeros_row,
                            const uint16_t *scale_col_1, const uint16_t *zeros_col_1,
                            const uint16_t *scale_col_2, const uint16_t *zeros_col_2, uint32_t rows,
                            uint32_t cols, uint16_t *x)
{
    for (uint32_t r = 0; r < rows; ++r)
        for (uint32_t c = 0; c < cols; ++c) {
            uint16_t sc = c == 0 ? scale_col_1[c] : scale_col_2[c];
            uint16_t zc = c == 0 ? zeros_col_1[c] : zeros_col_2[c];
            uint16_t e = int_to_half(q[(size_t)r * cols + c]);
            uint16_t inner = hsub(hsub(e, zeros_row[r]), zc);
            x[(size_t)r * cols + c] = hmul(hmul(scale_row[r], sc), inner);
        }
}

/* qlinear4bit/nn/linear.py:53-54 */
void duqo_add_bias(uint16_t *y, const uint16_t *bias, uint32_t rows, uint32_t cols)
{
    for (uint32_t r = 0; r < rows; ++r)
        for (uint32_t c = 0; c < cols; ++c) y[(size_t)r * cols + c] = hadd(y[(size_t)r * cols + c], bias[c]);
}

/* ---------------- 8-bit asymmetric layer (LinearQuant8bitASQ) ---------------- */

/* qlinear4bit/nn/quantizer.py:47-51, float32.  device_division != 0: scale = (max - min) * float32(1/127), the form
 * torch evaluates tensor / scalar in on a GPU; 0: the quotient (torch on a CPU). */
void duqo_asym8_scales_zeros(const float *x, uint32_t rows, uint32_t cols, int device_division, float *scale, float *zero)
{
    const volatile float inv = 1.0f / 127.0f;
    for (uint32_t r = 0; r < rows; ++r) {
        float mn = INFINITY, mx = -INFINITY;
        int nan = 0;
        for (uint32_t c = 0; c < cols; ++c) {
            float v = x[(size_t)r * cols + c];
            if (v != v) nan = 1;
            if (v < mn) mn = v;
            if (v > mx) mx = v;
        }
        if (nan) mn = mx = NAN;
        volatile float d = mx - mn;
        volatile float s = device_division ? d * inv : d / 127.0f;
        volatile float q = -mn / s;
        scale[r] = s;
        zero[r] = nearbyintf(q);
    }
}

/* src/kernels/quant.cu:244-264: the float quotient and the float zero point are converted to binary16 on their way
 * into __half2int_rn; the int add wraps; clamp to [0, 126] */
void duqo_asym_quant_8bit(const float *x, const float *scale, const float *zeros, uint32_t rows, uint32_t cols, int8_t *q)
{
    for (uint32_t r = 0; r < rows; ++r) {
        const int32_t zi = half_to_int_rn(duqo_f2h(zeros[r]));
        for (uint32_t c = 0; c < cols; ++c) {
            volatile float data = x[(size_t)r * cols + c] / scale[r];
            const int32_t qi = half_to_int_rn(duqo_f2h(data));
            const int32_t sum = (int32_t)((uint32_t)qi + (uint32_t)zi);
            q[(size_t)r * cols + c] = (int8_t)clampi(sum, 0, 126);
        }
    }
}

/* src/kernels/gemm.cu:46-81: A [M,K] x B [N,K]^T, int32 accumulation (wrapping) */
void duqo_matmul_s8(const int8_t *A, const int8_t *B, uint32_t M, uint32_t N, uint32_t K, int32_t *C)
{
#pragma omp parallel for
    for (uint32_t m = 0; m < M; ++m)
        for (uint32_t n = 0; n < N; ++n) {
            uint32_t acc = 0;
            for (uint32_t k = 0; k < K; ++k)
                acc += (uint32_t)((int32_t)A[(size_t)m * K + k] * (int32_t)B[(size_t)n * K + k]);
            C[(size_t)m * N + n] = (int32_t)acc;
        }
}

/* src/kernels/quant.cu:283-299: float32, one rounding per operator */
void duqo_asym_dequant_hprec(const int32_t *q, const float *scale_row, const float *zeros_row, const float *scale_col,
                             const float *zeros_col, uint32_t rows, uint32_t cols, float *x)
{
    for (uint32_t r = 0; r < rows; ++r)
        for (uint32_t c = 0; c < cols; ++c) {
            volatile float e = (float)q[(size_t)r * cols + c];
            volatile float scales = scale_row[r] * scale_col[c];
            volatile float zeros = zeros_row[r] + zeros_col[c];
            volatile float t = e - zeros;
            x[(size_t)r * cols + c] = scales * t;
        }
}
