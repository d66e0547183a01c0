// Per-token int4 quantizers for gfx950.
//
// Two families:
//  * given-scale kernels, one per reference launcher (sym, sym-dual, asym, asym-dual):
//    stream x once, 8 binary16 elements (one 128-bit load) -> one packed 32-bit word per
//    lane step, fully coalesced; a scalar kernel covers odd / unaligned shapes;
//  * fused row kernels that also compute the per-token scale (and zero): the row is
//    read from HBM once into registers, the |x| max (or min and max) is reduced with
//    wavefront shuffles (plus one LDS hop when several wavefronts share a row), and
//    the packed nibbles are written with 128-bit stores.
//
// Arithmetic follows the reference kernels operator by operator:
//   sym  : src/kernels/quant.cu:11-45     asym : src/kernels/quant.cu:99-132
//   dual : src/kernels/quant2.cu:9-45, 101-139
//   scale: qlinear4bit/nn/quantizer.py:13, 27-31
#include "duq_device.h"
#include "duq_launch.h"
#include "duq_rowquant.h"

namespace duq {

enum QuantKind { kSym = 0, kSymDual = 1, kAsym = 2, kAsymDual = 3 };

struct QuantParams {
    const uint16_t *x;
    const uint16_t *s1;  // scale / scale_1   [rows]
    const uint16_t *z1;  // zeros / zeros_1   [rows] (asym kinds)
    const uint16_t *s2;  // scale_2           [rows] (dual kinds)
    const uint16_t *z2;  // zeros_2           [rows] (asym dual)
    uint8_t *q;
    uint32_t rows, colsSrc, colsDst;
    int qmax;
};

// ---------------------------------------------------------------------------------
// scalar kernel: any shape, one thread per output byte (odd K, unaligned rows)
// ---------------------------------------------------------------------------------
template <int KIND>
__global__ __launch_bounds__(256) void quant_scalar_kernel(DUQ_HEAD_DECL, QuantParams tail)
{
    QuantParams p = with_head(tail, DUQ_HEAD_USE);
    to_global(p.x);
    to_global(p.s1);
    to_global(p.z1);
    to_global(p.s2);
    to_global(p.z2);
    to_global(p.q);
    const uint64_t total = (uint64_t)p.rows * p.colsDst;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (uint64_t)gridDim.x * blockDim.x) {
        const uint32_t row = (uint32_t)(i / p.colsDst);
        const uint32_t cd = (uint32_t)(i % p.colsDst);
        uint32_t byte = 0;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const uint32_t c = cd * 2 + e;
            if (c >= p.colsSrc) continue;
            const f16 xv = bits_to_f16(p.x[(uint64_t)row * p.colsSrc + c]);
            const bool first = c < (uint32_t)kQuantColK;
            uint32_t code;
            if (KIND == kSym) {
                code = sym_code(xv, row_rcp(bits_to_f16(p.s1[row])), p.qmax);
            } else if (KIND == kSymDual) {
                code = sym_code(xv, row_rcp(bits_to_f16(first ? p.s1[row] : p.s2[row])), p.qmax);
            } else if (KIND == kAsym) {
                code = asym_code(xv, row_rcp(bits_to_f16(p.s1[row])), rint_i32((float)bits_to_f16(p.z1[row])));
            } else {
                code = asym_pre_code(xv, row_rcp(bits_to_f16(first ? p.s1[row] : p.s2[row])),
                                     bits_to_f16(first ? p.z1[row] : p.z2[row]));
            }
            byte |= code << (4 * e);
        }
        p.q[i] = (uint8_t)byte;
    }
}

// ---------------------------------------------------------------------------------
// vector kernel: colsSrc % 8 == 0, x 16-byte aligned, q 4-byte aligned.
// One lane step = 8 elements in, one 32-bit word out; consecutive lanes take
// consecutive words, so loads are 1 KiB and stores 256 B contiguous per wavefront.
// ---------------------------------------------------------------------------------
template <int KIND>
__device__ __forceinline__ uint32_t quant8(const v4u raw, uint32_t col0, float r1, float r2, int qmax, int zi,
                                           f16 z1, f16 z2)
{
    uint32_t word = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const uint32_t w = raw[e >> 1];
        const f16 xv = bits_to_f16((uint16_t)((e & 1) ? (w >> 16) : (w & 0xFFFFu)));
        uint32_t code;
        if (KIND == kSym) {
            code = sym_code(xv, r1, qmax);
        } else if (KIND == kSymDual) {
            code = sym_code(xv, (col0 + e) < (uint32_t)kQuantColK ? r1 : r2, qmax);
        } else if (KIND == kAsym) {
            code = asym_code(xv, r1, zi);
        } else {
            const bool first = (col0 + e) < (uint32_t)kQuantColK;
            code = asym_pre_code(xv, first ? r1 : r2, first ? z1 : z2);
        }
        word |= code << (4 * e);
    }
    return word;
}

template <int KIND>
__global__ __launch_bounds__(256) void quant_vec_kernel(DUQ_HEAD_DECL, QuantParams tail)
{
    QuantParams p = with_head(tail, DUQ_HEAD_USE);
    to_global(p.x);
    to_global(p.s1);
    to_global(p.z1);
    to_global(p.s2);
    to_global(p.z2);
    to_global(p.q);
    const uint32_t vecPerRow = p.colsSrc >> 3;
    const uint64_t total = (uint64_t)p.rows * vecPerRow;
    const v4u *x4 = reinterpret_cast<const v4u *>(p.x);
    uint32_t *q32 = reinterpret_cast<uint32_t *>(p.q);
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (uint64_t)gridDim.x * blockDim.x) {
        const uint32_t row = (uint32_t)(i / vecPerRow);
        const uint32_t vec = (uint32_t)(i % vecPerRow);
        const v4u raw = __builtin_nontemporal_load(&x4[i]);
        const float r1 = row_rcp(bits_to_f16(p.s1[row]));
        float r2 = 0.f;
        int zi = 0;
        f16 z1 = (f16)0, z2 = (f16)0;
        if (KIND == kSymDual || KIND == kAsymDual) r2 = row_rcp(bits_to_f16(p.s2[row]));
        if (KIND == kAsym) zi = rint_i32((float)bits_to_f16(p.z1[row]));
        if (KIND == kAsymDual) {
            z1 = bits_to_f16(p.z1[row]);
            z2 = bits_to_f16(p.z2[row]);
        }
        q32[i] = quant8<KIND>(raw, vec * 8, r1, r2, p.qmax, zi, z1, z2);
    }
}

template <int KIND>
static int launch_quant(const QuantParams &p, hipStream_t stream)
{
    if (p.rows == 0 || p.colsSrc == 0) return 0;
    const bool vec_ok = (p.colsSrc % 8 == 0) && (reinterpret_cast<uintptr_t>(p.x) % 16 == 0) &&
                        (reinterpret_cast<uintptr_t>(p.q) % 4 == 0);
    if (vec_ok) {
        const uint64_t total = (uint64_t)p.rows * (p.colsSrc / 8);
        const uint32_t blocks = (uint32_t)std::min<uint64_t>((total + 255) / 256, 1u << 20);
        DUQ_LAUNCH_HEAD((quant_vec_kernel<KIND>), dim3(blocks), dim3(256), 0, stream, p);
    } else {
        const uint64_t total = (uint64_t)p.rows * p.colsDst;
        const uint32_t blocks = (uint32_t)std::min<uint64_t>((total + 255) / 256, 1u << 20);
        DUQ_LAUNCH_HEAD((quant_scalar_kernel<KIND>), dim3(blocks), dim3(256), 0, stream, p);
    }
    return (int)hipGetLastError();
}

int launch_sym_quant(const uint16_t *x, const uint16_t *scale, uint32_t rows, uint32_t colsSrc, uint32_t colsDst,
                     int qmax, uint8_t *q, hipStream_t stream)
{
    QuantParams p{x, scale, nullptr, nullptr, nullptr, q, rows, colsSrc, colsDst, qmax};
    return launch_quant<kSym>(p, stream);
}
int launch_sym_dual_quant(const uint16_t *x, const uint16_t *s1, const uint16_t *s2, uint32_t rows,
                          uint32_t colsSrc, uint32_t colsDst, int qmax, uint8_t *q, hipStream_t stream)
{
    QuantParams p{x, s1, nullptr, s2, nullptr, q, rows, colsSrc, colsDst, qmax};
    return launch_quant<kSymDual>(p, stream);
}
int launch_asym_quant(const uint16_t *x, const uint16_t *scale, const uint16_t *zeros, uint32_t rows,
                      uint32_t colsSrc, uint32_t colsDst, uint8_t *q, hipStream_t stream)
{
    QuantParams p{x, scale, zeros, nullptr, nullptr, q, rows, colsSrc, colsDst, 15};
    return launch_quant<kAsym>(p, stream);
}
int launch_asym_dual_quant(const uint16_t *x, const uint16_t *s1, const uint16_t *z1, const uint16_t *s2,
                           const uint16_t *z2, uint32_t rows, uint32_t colsSrc, uint32_t colsDst, uint8_t *q,
                           hipStream_t stream)
{
    QuantParams p{x, s1, z1, s2, z2, q, rows, colsSrc, colsDst, 15};
    return launch_quant<kAsymDual>(p, stream);
}

// ---------------------------------------------------------------------------------
// fused row kernels: scale (and zero) + quantize in one pass over x
// ---------------------------------------------------------------------------------
// A row of `cols` elements is split into units of 8 (one 128-bit load, one 32-bit store).
// WAVES wavefronts share one row; lane t owns units t, t+T, t+2T, ... (T = 64*WAVES), so
// every load and store instruction of a wavefront covers one contiguous 1 KB / 256 B span,
// and keeps up to kMaxUnits of them in registers between the reduction and the
// quantization: x is read from HBM exactly once.  Rows longer than 8*kMaxUnits*T elements
// run the same code with CACHED = false: the units are read a second time (from L2).
constexpr int kMaxUnits = 8;  // 64 elements = 32 VGPRs of row data per lane

// The fused row quantizer writes its codes / shadow with non-temporal stores (nobody reads them in this launch;
// measured at 2048 x 4096: shadow 6.6 against 7.15 us, nibbles level).
#ifndef DUQ_QUANT_NT_STORE
#define DUQ_QUANT_NT_STORE 1
#endif
#if DUQ_QUANT_NT_STORE
#define DUQ_QSTORE(ptr, val) __builtin_nontemporal_store((val), (ptr))
#else
#define DUQ_QSTORE(ptr, val) (*(ptr) = (val))
#endif

// The first 56 bytes (through qmax) reach the kernel in registers (DUQ_HEAD_DECL / with_head).
struct RowParams {
    const uint16_t *x;
    uint8_t *q;
    uint16_t *scale;
    uint16_t *zeros;
    uint8_t *bf6;     // BF6 kernels: E3M2 shadow of the codes, [rows][cols/32 x 16 B | cols/32 x 8 B]; q may be null
    uint32_t rows, cols;
    float clip;
    int qmax;
    int32_t *rowsum;  // asym only: non-null selects the signed-shifted form (code - 8, zero - 8, sum of codes)
};
static_assert(offsetof(RowParams, rowsum) == kHeadBytes, "the fields delivered in registers");

typedef _Float16 v32h __attribute__((ext_vector_type(32)));
typedef unsigned int v6u __attribute__((ext_vector_type(6)));

// 32 codes (four packed words, read as signed nibbles like the GEMM reads them) -> one E3M2
// block.  Position 8d + 2i + h of the block holds nibble i + 4h of word d: the pairing that
// costs one shift and one mask per two elements; the weight shadow uses the same order and
// the sum over k does not care.  0x6400 | u is the binary16 number 1024 + u, and the signed
// value of nibble n is (n ^ 8) - 8.
__device__ __forceinline__ v6u bf6_block(const uint32_t (&w)[4])
{
    typedef uint32_t v16u_t __attribute__((ext_vector_type(16)));
    v16u_t pairs;
    const v2h off = v2h{(f16)1032.0f, (f16)1032.0f};
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const uint32_t u = w[d] ^ 0x88888888u;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t bits = ((u >> (4 * i)) & 0x000F000Fu) | 0x64006400u;
            pairs[d * 4 + i] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(v2h, bits) - off);
        }
    }
    return __builtin_amdgcn_cvt_scalef32_pk32_bf6_f16(__builtin_bit_cast(v32h, pairs), 1.0f);
}

// BF6: the kernel also writes the E3M2 shadow of the codes (blocks of 32 elements = four
// consecutive units); the packed words of a row meet in LDS so that the loads keep the
// coalesced unit-per-lane pattern and a lane still converts whole blocks.  The packed nibbles
// are written only when p.q is given.
template <int WAVES, bool ASYM, bool CACHED, bool BF6 = false>
__global__ __launch_bounds__(WAVES * 64) void quantize_rows_kernel(DUQ_HEAD_DECL, RowParams tail)
{
    RowParams p = with_head(tail, DUQ_HEAD_USE);
    to_global(p.x);
    to_global(p.q);
    to_global(p.scale);
    to_global(p.zeros);
    to_global(p.bf6);
    constexpr int T = WAVES * 64;
    __shared__ float red[3][WAVES];
    __shared__ int red_sum[WAVES];
    const bool shifted = ASYM && p.rowsum != nullptr;
    int code_sum = 0;  // sum of this lane's unsigned codes (shifted form only)
    const uint32_t row = blockIdx.x;
    const uint32_t tid = threadIdx.x;
    const uint32_t nunits = p.cols >> 3;  // units of 8 elements
    const v4u *xrow = reinterpret_cast<const v4u *>(p.x + (uint64_t)row * p.cols);
    uint32_t *qrow = reinterpret_cast<uint32_t *>(p.q + (uint64_t)row * (p.cols >> 1));
    __shared__ __attribute__((aligned(16))) uint32_t words[BF6 && CACHED ? T * kMaxUnits : 4];
    // unit held in register slot i
    auto unit_of = [&](int i) -> uint32_t { return tid + i * T; };

    v4u regs[kMaxUnits];
    PkMinMax st;  // packed running maximum and minimum of this lane's elements

    auto reduce_unit = [&](const v4u &g) { st.add8(g); };

    if (CACHED) {
#pragma unroll
        for (int i = 0; i < kMaxUnits; ++i) {
            const uint32_t u = unit_of(i);
            regs[i] = u < nunits ? __builtin_nontemporal_load(&xrow[u]) : v4u{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int i = 0; i < kMaxUnits; ++i)
            if (unit_of(i) < nunits) reduce_unit(regs[i]);
    } else {
        for (uint32_t u = tid; u < nunits; u += T) reduce_unit(xrow[u]);
    }

    // ---- row reduction: DPP steps inside a wavefront, one LDS hop across wavefronts ----
    float a, b = 0.f;
    uint32_t m16;  // largest |x| bit pattern; above 0x7C00: a NaN (which fminf / fmaxf would drop)
    if (!ASYM) {
        m16 = wave_max_u32(st.absmax_bits());
        a = __builtin_bit_cast(float, m16);  // carried as raw bits
    } else {
        st.wave_reduce();
        m16 = st.absmax_bits();
        a = st.min_f32();
        b = st.max_f32();
    }
    if (WAVES > 1) {
        const uint32_t wave = tid >> 6;
        if ((tid & 63u) == 0) {
            red[0][wave] = a;
            red[1][wave] = b;
            red[2][wave] = __builtin_bit_cast(float, m16);
        }
        __syncthreads();
        if (!ASYM) {
            uint32_t m = 0;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) m = max(m, __builtin_bit_cast(uint32_t, red[0][w]));
            a = __builtin_bit_cast(float, m);
        } else {
            a = red[0][0];
            b = red[1][0];
            m16 = __builtin_bit_cast(uint32_t, red[2][0]);
#pragma unroll
            for (int w = 1; w < WAVES; ++w) {
                a = fminf(a, red[0][w]);
                b = fmaxf(b, red[1][w]);
                m16 = max(m16, __builtin_bit_cast(uint32_t, red[2][w]));
            }
        }
    }
    if (ASYM && m16 > 0x7C00u) a = b = __builtin_nanf("");  // torch's min / max return NaN for a row that holds one

    // ---- per-token scale / zero and the quantization constants (duq_rowquant.h) ----
    RowQuant<ASYM> rq;
    rq.init(__builtin_bit_cast(uint32_t, a) & 0xFFFFu, a, b, p.clip, p.qmax);
    if (tid == 0) {
        p.scale[row] = f16_to_bits(rq.s);
        if (ASYM) p.zeros[row] = f16_to_bits(shifted ? rq.z - (f16)8.0f : rq.z);
    }

    // ---- quantize + pack: 8 elements -> one 32-bit store ----
    auto quant_unit = [&](const v4u &g) -> uint32_t {
        uint32_t w = rq.quant8(g);
        if (shifted) {
            // eight unsigned codes: sum them, then u - 8 as a signed nibble is u with bit 3 flipped
            const uint32_t pairs = (w & 0x0F0F0F0Fu) + ((w >> 4) & 0x0F0F0F0Fu);
            code_sum = (int)__builtin_amdgcn_udot4(pairs, 0x01010101u, (uint32_t)code_sum, false);
            w ^= 0x88888888u;
        }
        return w;
    };
    if (BF6) {
        // cols % 32 == 0: a block is all inside the row or all outside
        const uint32_t nblk = p.cols >> 5;
        uint8_t *srow = p.bf6 + (uint64_t)row * nblk * 24;
        auto put_block = [&](uint32_t b, const uint32_t (&w)[4]) {
            if (p.q) DUQ_QSTORE(reinterpret_cast<v4u *>(qrow + 4 * b), (v4u{w[0], w[1], w[2], w[3]}));
            const v6u f = bf6_block(w);
            DUQ_QSTORE(reinterpret_cast<v4u *>(srow + b * 16), (v4u{f[0], f[1], f[2], f[3]}));
            DUQ_QSTORE(reinterpret_cast<v2u *>(srow + nblk * 16 + b * 8), (v2u{f[4], f[5]}));
        };
        if (CACHED) {
#pragma unroll
            for (int i = 0; i < kMaxUnits; ++i) {
                const uint32_t u = tid + i * T;
                if (u < nunits) {
                    const uint32_t w = quant_unit(regs[i]);
                    words[u] = w;
                    if (p.q) DUQ_QSTORE(&qrow[u], w);
                }
            }
            __syncthreads();
#pragma unroll
            for (int g = 0; g < kMaxUnits / 4; ++g) {
                const uint32_t b = tid + g * T;
                if (b < nblk) {
                    const v4u w4 = *reinterpret_cast<const v4u *>(&words[4 * b]);
                    const uint32_t w[4] = {w4[0], w4[1], w4[2], w4[3]};
                    const v6u f = bf6_block(w);
                    DUQ_QSTORE(reinterpret_cast<v4u *>(srow + b * 16), (v4u{f[0], f[1], f[2], f[3]}));
                    DUQ_QSTORE(reinterpret_cast<v2u *>(srow + nblk * 16 + b * 8), (v2u{f[4], f[5]}));
                }
            }
        } else {
            for (uint32_t b = tid; b < nblk; b += T) {
                uint32_t w[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) w[j] = quant_unit(xrow[4 * b + j]);
                put_block(b, w);
            }
        }
    } else if (CACHED) {
#pragma unroll
        for (int i = 0; i < kMaxUnits; ++i) {
            const uint32_t u = tid + i * T;
            if (u < nunits) DUQ_QSTORE(&qrow[u], quant_unit(regs[i]));
        }
    } else {
        for (uint32_t u = tid; u < nunits; u += T) DUQ_QSTORE(&qrow[u], quant_unit(xrow[u]));
    }
    if (shifted) {  // uniform branch: sum of (u - 8) over the row
        code_sum = wave_sum_i32(code_sum);
        if (WAVES > 1) {
            if ((tid & 63u) == 0) red_sum[tid >> 6] = code_sum;
            __syncthreads();
            code_sum = 0;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) code_sum += red_sum[w];
        }
        if (tid == 0) p.rowsum[row] = code_sum - 8 * (int)p.cols;
    }
}

template <bool ASYM>
static int launch_rows(const RowParams &p, hipStream_t stream)
{
    if (p.rows == 0 || p.cols == 0) return 0;
    const uint32_t nunits = p.cols / 8;
    const dim3 grid(p.rows);
    // Wavefronts per row: enough that a lane holds at most `per_lane` units.  Four units per
    // lane stream best when the grid is large; smaller grids are latency-bound and spread a
    // row over more lanes (2, then 1 unit each) to shorten every lane's serial work.
    auto waves_for = [&](uint32_t per_lane) {
        uint32_t w = 1;
        while (w < 16 && w * 64 * per_lane < nunits) w *= 2;
        return w;
    };
    uint32_t waves = waves_for(4);
    if ((uint64_t)p.rows * waves < 2048) waves = waves_for(2);
    if ((uint64_t)p.rows * waves < 512) waves = waves_for(1);
    const bool cached = waves * 64 * kMaxUnits >= nunits;
#define DUQ_ROWS_LAUNCH(W, C)                                                                                \
    if (p.bf6)                                                                                               \
        DUQ_LAUNCH_HEAD((quantize_rows_kernel<W, ASYM, C, true>), grid, dim3(W * 64), 0, stream, p);      \
    else                                                                                                     \
        DUQ_LAUNCH_HEAD((quantize_rows_kernel<W, ASYM, C, false>), grid, dim3(W * 64), 0, stream, p);
#define DUQ_ROWS_CASE(W)                                                                                     \
    case W:                                                                                                  \
        if (cached) {                                                                                        \
            DUQ_ROWS_LAUNCH(W, true)                                                                         \
        } else {                                                                                             \
            DUQ_ROWS_LAUNCH(W, false)                                                                        \
        }                                                                                                    \
        break;
    switch (waves) {
        DUQ_ROWS_CASE(1)
        DUQ_ROWS_CASE(2)
        DUQ_ROWS_CASE(4)
        DUQ_ROWS_CASE(8)
        DUQ_ROWS_CASE(16)
    }
#undef DUQ_ROWS_CASE
#undef DUQ_ROWS_LAUNCH
    return (int)hipGetLastError();
}

int launch_quantize_rows_sym(const uint16_t *x, uint32_t rows, uint32_t cols, float clip, int qmax, uint8_t *q,
                             uint16_t *scale, uint8_t *bf6, hipStream_t stream)
{
    RowParams p{x, q, scale, nullptr, bf6, rows, cols, clip, qmax, nullptr};
    return launch_rows<false>(p, stream);
}
int launch_quantize_rows_asym(const uint16_t *x, uint32_t rows, uint32_t cols, uint8_t *q, uint16_t *scale,
                              uint16_t *zeros, int32_t *rowsum, uint8_t *bf6, hipStream_t stream)
{
    RowParams p{x, q, scale, zeros, bf6, rows, cols, 1.0f, 15, rowsum};
    return launch_rows<true>(p, stream);
}

}  // namespace duq
