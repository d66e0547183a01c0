// Decode kernels (M <= 64 activation rows, K <= 16384): weight streaming for problems of a few MB,
// where a launch lives for two or three microseconds and what counts is that every byte is requested
// in the kernel's first instructions and nothing else sits on the critical path.
//
//   C[m,n] = sum_k s4(A[m,k]) * s4(B[n,k])        (src/kernels/gemm.cu:8-43 of the reference, at M <= 16)
//
// Both kernels
//  * issue every weight load of the workgroup before anything else (no ring: the whole share of a
//    workgroup, 16-32 KB, is in flight at once),
//  * fetch the epilogue parameters of the outputs a lane will store right behind them, so that no
//    dependent memory round trip follows the arithmetic,
//  * take the activations pre-quantized (packed nibbles, the reference's operator boundary); the rows kernel
//    also takes them as binary16 (FUSEQ): the workgroup then computes the per-token scales and codes itself
//    while its weights are in flight (SymQuantizer.forward, qlinear4bit/nn/quantizer.py:10-16, and
//    src/kernels/quant.cu:11-45, through the same RowQuant code as the stand-alone quantizer), which makes
//    quantize + GEMM + dequant one launch.  (Up to four rows only: every workgroup reads all the rows, and from
//    eight rows on that is more bytes into a CU than its share of the weights.)
//
//  rows kernel (M <= 4): v_dot8_i32_i4 on the packed nibbles.  A wavefront owns four weight rows and the
//    whole K range: lane l holds bytes [i*1024 + l*16, +16) of each row, so a load instruction covers 1 KB
//    of one row and an activation register serves four rows.  The 4*M partial sums of a lane meet the other
//    lanes' through the wavefront's own piece of LDS (no barrier) and a few DPP steps.
//  MFMA kernel (5 <= M <= 64): v_mfma_i32_16x16x64_i8, eight wavefronts split K for one 16-column tile, one to
//    four tiles of 16 rows against the same weight fragments, the partial tiles meet in LDS, 256 threads finish
//    one output each per row tile; one round of at most 256 workgroups with several column tiles each.
#include <cstddef>

#include "duq_epilogue.h"
#include "duq_launch.h"
#include "duq_rowquant.h"
#include "duq_tiles.h"

// Wavefronts per workgroup of the rows kernel when it quantizes its rows itself (binary16 in).  The quantize phase is
// vector arithmetic (about 27 instructions per eight elements), the same for every workgroup, and sits between the
// arrival of the activations and the dot products: a wavefront alone on its SIMD issues it at half the rate that
// two reach together.  Measured (us, N = K = 4096 unless said): two rows 3.25 with four wavefronts, 3.21 with eight;
// three / four rows 4.11 / 4.17 with four, 3.67 / 3.68 with eight (and with sixteen); four rows of 8192 / 11008
// elements 7.5 / 8.9 with four, 6.5 / 7.1 with sixteen; eight rows 5.0 with eight, 5.1 with sixteen, of 8192
// elements 9.1 with eight, 8.7 with sixteen.
#ifndef DUQ_DEC_FUSEQ_WAVES
#define DUQ_DEC_FUSEQ_WAVES 8     // eight rows; and several tiles per workgroup
#endif
#ifndef DUQ_DEC_FUSEQ_WAVES_M4
#define DUQ_DEC_FUSEQ_WAVES_M4 8  // three or four rows of up to 4096 elements
#endif
#ifndef DUQ_DEC_FUSEQ_WAVES_M4L
#define DUQ_DEC_FUSEQ_WAVES_M4L 16  // of more
#endif
#ifndef DUQ_DEC_FUSEQ_WAVES_M8L
#define DUQ_DEC_FUSEQ_WAVES_M8L 16  // eight rows of more than 4096 elements
#endif
#ifndef DUQ_DEC_FUSEQ_WAVES_M2
#define DUQ_DEC_FUSEQ_WAVES_M2 4
#endif
#ifndef DUQ_DEC_R
#define DUQ_DEC_R 4
#endif
// Cache policy of the rows kernel's weight loads (and of the read probe that mirrors them): 2 = non-temporal.  A
// load instruction of that kernel covers whole cache lines that nobody reads again (measured, one row: N = K = 4096
// 3.00 against 3.08 us, N = 28672 K = 8192 19.6 against 21.2).  The MFMA kernel reads a line in two instructions (64
// bytes of a row each) and loses with it (16 rows, N = K = 4096: 4.13 against 3.90 us): it keeps the default.
#ifndef DUQ_DEC_WLOAD_AUX
#define DUQ_DEC_WLOAD_AUX 2
#endif
#ifndef DUQ_DEC_WAVES
#define DUQ_DEC_WAVES 8
#endif
// 8-element units whose quantization chains are interleaved in the kernels that quantize their rows themselves
#ifndef DUQ_DEC_QUANT_GROUP
#define DUQ_DEC_QUANT_GROUP 8
#endif
// wavefronts per workgroup of the MFMA kernel when it quantizes its 16 rows itself
// (16 rows, N = 4096: sixteen against eight wavefronts K = 4096 7.2 against 7.9 us, K = 2048 4.9 against 5.4)
#ifndef DUQ_DEC_MFMA_FUSEQ_WAVES
#define DUQ_DEC_MFMA_FUSEQ_WAVES 16
#endif

namespace duq {

namespace {

constexpr uint32_t kNibbleMaskD = 0xF0F0F0F0u;

// The first 56 bytes (through `y`) reach the kernels in registers (DUQ_HEAD_DECL / with_head).
struct DecodeParams {
    const uint8_t *A;    // packed activations [M, K/2] (pre-quantized input)
    const uint16_t *X;   // binary16 activations [M, K] (FUSEQ)
    const uint8_t *B;    // packed weights [N, K/2]
    uint32_t M, N, K;
    uint32_t tiles_per_wg;
    int32_t *C;          // int32 out (EPI < 0)
    uint16_t *y;         // binary16 out (EPI >= 0)
    Epilogue epi;        // FUSEQ: s_row is not read, the kernel computes it
    float clip;          // FUSEQ
    int qmax;            // FUSEQ
    uint8_t *q_out;      // FUSEQ, optional: the packed codes [M, K/2] (written by workgroup 0)
    uint16_t *s_out;     // FUSEQ, optional: the per-token scales [M]
    uint16_t *z_out;     // FUSEQ with an asymmetric epilogue, optional: the per-token zero points [M]
    int32_t *rs_out;     // FUSEQ with the row-sum epilogue, optional: the per-token sums of the shifted codes [M]
};
static_assert(offsetof(DecodeParams, y) + sizeof(uint16_t *) == kHeadBytes, "the fields delivered in registers");

// The quantization step over N units, G at a time (RowQuant::quant_units: the path is chosen once per group and the
// group's chains interleave; a group holds 4 G more registers than a single unit).
template <int G, int S = 0, bool ASYM, int N>
__device__ __forceinline__ void quant_in_groups(const RowQuant<ASYM> &rq, const v4u (&raw)[N], uint32_t (&out)[N])
{
    if constexpr (S < N) {
        constexpr int L = N - S < G ? N - S : G;
        v4u in[L];
        uint32_t w[L];
#pragma unroll
        for (int j = 0; j < L; ++j) in[j] = raw[S + j];
        rq.quant_units(in, w);
#pragma unroll
        for (int j = 0; j < L; ++j) out[S + j] = w[j];
        quant_in_groups<G, S + L>(rq, raw, out);
    }
}

template <int CTRL>
__device__ __forceinline__ int dpp_add(int v)
{
    return v + __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}
// Sum over groups of G consecutive lanes (G = 2, 4, 8 or 16, inside one DPP row): every lane of a group
// ends with the group's total.
template <int G>
__device__ __forceinline__ int group_sum(int v)
{
    v = dpp_add<0xB1>(v);               // quad_perm [1,0,3,2]
    if (G >= 4) v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
    if (G >= 8) v = dpp_add<0x141>(v);  // row_half_mirror: lane i <- lane 7 - i
    if (G >= 16) v = dpp_add<0x140>(v); // row_mirror: lane i <- lane 15 - i
    return v;
}

__device__ __forceinline__ v4u load16(const void *p) { return *reinterpret_cast<const v4u *>(p); }

// Epilogue records of one output row / one output column, by mode: modes 0..4 the shared ColParams / RowEpi,
// mode 5 (row-sum epilogue of the dual-uniform layer) the records that also carry the codes of input columns 0..9.
template <int MODE>
struct EpiRec {
    using Col = ColParams;
    using Row = RowEpi;
};
template <>
struct EpiRec<5> {
    using Col = DualCol;
    using Row = DualRow;
};

// B / A: the packed operands (mode 5 reads the first eight bytes of the row)
template <int MODE>
__device__ __forceinline__ typename EpiRec<MODE>::Col load_col_rt(const Epilogue &e, uint32_t col, bool bias, const uint8_t *B,
                                                                  uint32_t kbytes)
{
    if constexpr (MODE == 5)
        return load_dual_col(e, B, kbytes, col, bias);
    else
        return bias ? load_col<MODE, true>(e.s_col_1, e.z_col_1, e.s_col_2, e.z_col_2, e.bias, col, e.rs_col)
                    : load_col<MODE, false>(e.s_col_1, e.z_col_1, e.s_col_2, e.z_col_2, e.bias, col, e.rs_col);
}
template <int MODE>
__device__ __forceinline__ typename EpiRec<MODE>::Row load_row_rt(const Epilogue &e, uint32_t row, const uint8_t *A, uint32_t kbytes)
{
    if constexpr (MODE == 5)
        return load_dual_row(e, A, kbytes, row);
    else
        return load_row<MODE>(e, row);
}
template <int MODE>
__device__ __forceinline__ uint16_t dequant_rt(int acc, const typename EpiRec<MODE>::Row &r, const typename EpiRec<MODE>::Col &c,
                                               bool bias)
{
    if constexpr (MODE == 5)
        return dual_finish(acc, r, c, bias);
    else
        return bias ? dequant_one<MODE, true>(acc, r, c) : dequant_one<MODE, false>(acc, r, c);
}

// ---------------------------------------------------------------------------------
// rows kernel: M <= MR <= 4 (8 with binary16 activations quantized inside), K <= XS * 2048
// ---------------------------------------------------------------------------------
// WAVES wavefronts of R = 16 / WAVES weight rows each: 16 weight rows ("a tile") per workgroup either way.  Eight
// wavefronts help when the workgroup quantizes four activation rows itself and a CU holds several workgroups
// (launcher).  MULTI: a workgroup owns p.tiles_per_wg consecutive tiles and keeps two tiles' weights in flight
// (two register sets that alternate), so that a launch is one round of at most 256 workgroups: the activations
// are fetched, and with FUSEQ quantized, once per CU and not once per tile.
template <int MR, int XS, bool FUSEQ, int EPI, int WAVES = 4, bool MULTI = false>
__global__ __launch_bounds__(WAVES * 64) void gemv_s4_rows_kernel(DUQ_HEAD_DECL, DecodeParams tail)
{
    const DecodeParams p = with_head(tail, DUQ_HEAD_USE);
    constexpr int R = 4 * DUQ_DEC_R / WAVES;  // weight rows per wavefront
    constexpr int V = MR * R;        // partial sums per lane: 4, 8 or 16
    constexpr int LPV = 64 / V;      // lanes that finish one sum: 16, 8 or 4
    constexpr int MODE = EPI < 0 ? 0 : EPI;
    constexpr uint32_t XSTRIDE = XS * 1024;
    static_assert(MR == 1 || MR == 2 || MR == 4 || (MR == 8 && WAVES >= 8), "rows");
    static_assert(WAVES == 4 || WAVES == 8 || WAVES == 16, "wavefronts per workgroup");
    static_assert(V >= 4 && V <= 16 && (XS * MR * 4) % WAVES == 0, "partial sums per lane, quantize units per lane");
    __shared__ __attribute__((aligned(16))) int red[WAVES][V * 64];
    __shared__ __attribute__((aligned(16))) uint8_t xs[FUSEQ ? MR * XSTRIDE : 16];
    __shared__ uint32_t rmax[WAVES];
    __shared__ float rlo[WAVES], rhi[WAVES];
    __shared__ int rsum[WAVES];
    __shared__ uint16_t srow[MR], zrow[MR];
    __shared__ int rsrow[MR];
    // binary16 rows in: the epilogue decides the quantizer (SymQuantizer for the symmetric epilogues, AsymQuantizer
    // for the asymmetric ones; the row-sum epilogue takes the signed-shifted codes, code - 8 and zero - 8, and the
    // per-token sum of the shifted codes)
    constexpr bool ASYMQ = FUSEQ && (MODE == 1 || MODE == 3 || MODE == 4 || MODE == 5);
    constexpr bool SHIFTQ = FUSEQ && (MODE == 4 || MODE == 5);
    using ColRec = typename EpiRec<MODE>::Col;
    using RowRec = typename EpiRec<MODE>::Row;

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t kbytes = p.K >> 1;
    const uint32_t tile0 = MULTI ? blockIdx.x * p.tiles_per_wg : blockIdx.x;
    const uint32_t tile_end = MULTI ? min(tile0 + p.tiles_per_wg, (p.N + 4 * DUQ_DEC_R - 1) / (4 * DUQ_DEC_R)) : tile0 + 1;

    // ---- loads, in the order their data is needed (loads return in order: waiting for one waits for every
    // earlier one): the activations first, then every weight byte of this wavefront's first tile, then the
    // parameters of the output this lane will finish
    // activations: lane l needs bytes [i*1024 + l*16, +16) of every row
    v4u xr[MR][XS];
    constexpr int WPR = WAVES / MR;           // wavefronts that share a row in the quantize phase
    constexpr int UPL = FUSEQ ? XS * MR * 4 / WAVES : 1;  // 8-element units per lane in the quantize phase
    const uint32_t qrow = wave / WPR, qpart = wave % WPR;
    v4u raw[UPL];
    const uint32_t nunits = p.K >> 3;
    if (!FUSEQ) {
        const __amdgpu_buffer_rsrc_t rX = make_rsrc(p.A, p.M * kbytes);  // rows past M read as zero
#pragma unroll
        for (int m = 0; m < MR; ++m)
#pragma unroll
            for (int i = 0; i < XS; ++i) {
                const uint32_t off = i * 1024 + lane * 16;
                xr[m][i] = buf_load16(rX, off < kbytes ? m * kbytes + off : kOobOffset, 0);
            }
    } else {
        // the workgroup quantizes the MR rows into LDS: WPR = WAVES / MR wavefronts share a row, wavefront `part` of
        // a row owns its 8-element units part*64 + lane, + 64*WPR, ...
        const __amdgpu_buffer_rsrc_t rX = make_rsrc(p.X, p.M * p.K * 2);  // rows past M read as zero
#pragma unroll
        for (int j = 0; j < UPL; ++j) {
            const uint32_t c = qpart * 64 + lane + j * (64 * WPR);
            raw[j] = buf_load16(rX, c < nunits ? (qrow * p.K + c * 8) * 2 : kOobOffset, 0);
        }
    }
    // Eight wavefronts that quantize: all of them request their activations before any requests weights (the CU
    // serves requests in order, and a wavefront whose activations queue behind another's weights holds up the
    // whole workgroup at the staging barrier below; measured at 8 rows, K = 4096: N = 4096 5.6 against 6.2 us,
    // N = 11008 8.2 against 8.5; with four wavefronts it changes nothing)
    if (FUSEQ && WAVES >= 8) __builtin_amdgcn_s_barrier();
    const __amdgpu_buffer_rsrc_t rW = make_rsrc(p.B, p.N * kbytes);
    // the weights of tile t for this wavefront (tiles past the workgroup's last read as zero, unused)
    auto load_w = [&](uint32_t tile, v4u(&w)[R][XS]) {
        const uint32_t n0 = (tile * WAVES + wave) * R;
        const uint32_t nrows = (!MULTI || tile < tile_end) ? p.N : 0u;
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int i = 0; i < XS; ++i) {
                const uint32_t off = i * 1024 + lane * 16;
                // K % 64 == 0: a 16-byte piece is all in or all out
                const bool ok = off < kbytes && n0 + r < nrows;
                w[r][i] = __builtin_bit_cast(
                    v4u, __builtin_amdgcn_raw_buffer_load_b128(rW, (int)(ok ? (n0 + r) * kbytes + off : kOobOffset), 0, DUQ_DEC_WLOAD_AUX));
            }
    };
    v4u w0[R][XS], w1[MULTI ? R : 1][MULTI ? XS : 1];
    load_w(tile0, w0);
    const uint32_t myv = lane / LPV, sub = lane % LPV;
    const uint32_t my_m = myv / R, my_r = wave * R + myv % R;  // my_r: weight row inside a tile
    const bool bias = p.epi.bias != nullptr;
    auto load_cp = [&](uint32_t tile) {
        ColRec c{};
        if (EPI >= 0) c = load_col_rt<MODE>(p.epi, min(tile * (4 * DUQ_DEC_R) + my_r, p.N - 1), bias, p.B, kbytes);
        return c;
    };
    ColRec cp = load_cp(tile0);
    RowRec rp{};
    if (EPI >= 0 && !FUSEQ) rp = load_row_rt<MODE>(p.epi, min(my_m, p.M - 1), p.A, kbytes);

    // what the quantize phase needs of the kernel arguments, fetched here under the vector loads above: a scalar
    // load issued where the value is first used (the compiler sinks it into the branch that uses it) is waited for on
    // its own, and a fetch of kernel arguments costs about half a microsecond (measured: 4 rows, N = K = 4096, 5.5
    // against 4.9 us)
    const float q_clip = p.clip;
    const int q_qmax = p.qmax;
    uint8_t *const q_out = p.q_out;
    uint16_t *const s_out = p.s_out, *const z_out = p.z_out;
    int32_t *const rs_out = p.rs_out;
    if (FUSEQ)
        asm volatile("" ::"s"(q_clip), "s"(q_qmax), "s"(q_out), "s"(s_out), "s"(z_out), "s"(rs_out));
    // (the output pointers arrive in registers)
    const auto c_out = as_global(p.C);
    const auto y_out = as_global(p.y);

    if (FUSEQ) {
        // statistics of this wavefront's share of its row.  Units past the row end read as zero: that changes no
        // maximum of |x|, but it would change a minimum or a maximum, so the asymmetric form skips them.
        PkMinMax st;
#pragma unroll
        for (int j = 0; j < UPL; ++j)
            if (!ASYMQ || qpart * 64 + lane + j * (64 * WPR) < nunits) st.add8(raw[j]);
        uint32_t m16;
        float lo = 0.f, hi = 0.f;
        if (!ASYMQ) {
            m16 = wave_max_u32(st.absmax_bits());
        } else {
            st.wave_reduce();
            m16 = st.absmax_bits();
            lo = st.min_f32();
            hi = st.max_f32();
        }
        if (WPR > 1) {  // the row's statistics cross its wavefronts through LDS
            if (lane == 0) {
                rmax[wave] = m16;
                if (ASYMQ) {
                    rlo[wave] = lo;
                    rhi[wave] = hi;
                }
            }
            __syncthreads();
            m16 = rmax[qrow * WPR];
            if (ASYMQ) {
                lo = rlo[qrow * WPR];
                hi = rhi[qrow * WPR];
            }
#pragma unroll
            for (int i = 1; i < WPR; ++i) {
                m16 = max(m16, rmax[qrow * WPR + i]);
                if (ASYMQ) {
                    lo = fminf(lo, rlo[qrow * WPR + i]);
                    hi = fmaxf(hi, rhi[qrow * WPR + i]);
                }
            }
        }
        if (ASYMQ && m16 > 0x7C00u) lo = hi = __builtin_nanf("");  // torch's min / max return NaN for a row that holds one
        int code_sum = 0;
        // rows past M (the last rows of the MR the kernel is built for) are neither quantized nor used
        if (qrow < p.M) {
            RowQuant<ASYMQ> rq;
            rq.init(m16, lo, hi, q_clip, q_qmax);
            const bool copy_out = blockIdx.x == 0;
            uint32_t words[UPL];
            quant_in_groups<(XS >= 8 ? 4 : DUQ_DEC_QUANT_GROUP)>(rq, raw, words);  // (long rows: registers)
#pragma unroll
            for (int j = 0; j < UPL; ++j) {
                const uint32_t c = qpart * 64 + lane + j * (64 * WPR);
                if (c < nunits) {
                    uint32_t word = words[j];
                    if (SHIFTQ) {
                        // eight unsigned codes: sum them, then u - 8 as a signed nibble is u with bit 3 flipped
                        const uint32_t pairs = (word & 0x0F0F0F0Fu) + ((word >> 4) & 0x0F0F0F0Fu);
                        code_sum = (int)__builtin_amdgcn_udot4(pairs, 0x01010101u, (uint32_t)code_sum, false);
                        word ^= 0x88888888u;
                    }
                    *reinterpret_cast<uint32_t *>(xs + qrow * XSTRIDE + c * 4) = word;
                    if (copy_out && q_out) reinterpret_cast<uint32_t *>(q_out + (uint64_t)qrow * kbytes)[c] = word;
                }
            }
            if (SHIFTQ) {
                code_sum = wave_sum_i32(code_sum);
                if (lane == 0) rsum[wave] = code_sum;
            }
            if (qpart == 0 && lane == 0) {
                const f16 z = SHIFTQ ? rq.z - (f16)8.0f : rq.z;
                srow[qrow] = f16_to_bits(rq.s);
                if (ASYMQ) zrow[qrow] = f16_to_bits(z);
                if (copy_out && s_out) s_out[qrow] = f16_to_bits(rq.s);
                if (ASYMQ && copy_out && z_out) z_out[qrow] = f16_to_bits(z);
            }
        }
        __syncthreads();
        if (SHIFTQ) {
            // per-token sum of the shifted codes: the parts of a row's wavefronts, minus 8 per element
            if (tid < (uint32_t)MR && tid < p.M) {
                int t = -8 * (int)p.K;
#pragma unroll
                for (int i = 0; i < WPR; ++i) t += rsum[tid * WPR + i];
                rsrow[tid] = t;
                if (blockIdx.x == 0 && rs_out) rs_out[tid] = t;
            }
            __syncthreads();
        }
        // (bytes past the row end are never written: the weights read as zero there)
#pragma unroll
        for (int m = 0; m < MR; ++m)
#pragma unroll
            for (int i = 0; i < XS; ++i) xr[m][i] = load16(xs + m * XSTRIDE + i * 1024 + lane * 16);
        const uint32_t rm = min(my_m, (uint32_t)MR - 1);
        if constexpr (MODE == 5) {
            // the row record from the codes this workgroup just wrote
            const v2u head = *reinterpret_cast<const v2u *>(xs + rm * XSTRIDE);
            rp.xlo = head[0];
            rp.xhi = head[1] & 0xFFu;
            rp.zx = (uint32_t)rint_i32((float)bits_to_f16(zrow[rm]));
            rp.sx = (float)bits_to_f16(srow[rm]);
            rp.rxl = dual_head_sum(rp.xlo, rp.xhi);
            rp.rxr = (uint32_t)rsrow[rm] - rp.rxl;
        } else {
            rp.s = bits_to_f16(srow[rm]);
            if (ASYMQ) rp.z = bits_to_f16(zrow[rm]);
            if (SHIFTQ) rp.rs = rsrow[rm];
        }
    }

    auto do_tile = [&](uint32_t tile, const v4u(&w)[R][XS], const ColRec &c) {
        // ---- dot products on the packed nibbles
        int acc[MR][R];
#pragma unroll
        for (int m = 0; m < MR; ++m)
#pragma unroll
            for (int r = 0; r < R; ++r) acc[m][r] = 0;
#pragma unroll
        for (int i = 0; i < XS; ++i)
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int m = 0; m < MR; ++m)
#pragma unroll
                    for (int d = 0; d < 4; ++d)
                        acc[m][r] = __builtin_amdgcn_sdot8((int)w[r][i][d], (int)xr[m][i][d], acc[m][r], false);

        // ---- the V sums of 64 lanes each: through this wavefront's piece of LDS (a wavefront's LDS operations
        // execute in order: no barrier), V entries per lane back, then log2(LPV) DPP steps
        int *mine = red[wave];
#pragma unroll
        for (int v = 0; v < V; ++v) mine[v * 64 + lane] = acc[v / R][v % R];
        __builtin_amdgcn_wave_barrier();
        int sum = 0;
#pragma unroll
        for (int e = 0; e < V / 4; ++e) {
            const v4i t = *reinterpret_cast<const v4i *>(&mine[lane * V + e * 4]);  // = [myv * 64 + sub * V + e * 4]
            sum += (t[0] + t[1]) + (t[2] + t[3]);
        }
        __builtin_amdgcn_wave_barrier();
        sum = group_sum<LPV>(sum);
        const uint32_t my_n = tile * (4 * DUQ_DEC_R) + my_r;
        if (sub == 0 && my_m < p.M && my_n < p.N) {
            if (EPI < 0)
                c_out[(uint64_t)my_m * p.N + my_n] = sum;
            else
                y_out[(uint64_t)my_m * p.N + my_n] = dequant_rt<MODE>(sum, rp, c, bias);
        }
    };

    if constexpr (!MULTI) {
        do_tile(tile0, w0, cp);
    } else {
        for (uint32_t t = tile0; t < tile_end; t += 2) {
            load_w(t + 1, w1);
            const ColRec cp1 = load_cp(t + 1 < tile_end ? t + 1 : t);
            do_tile(t, w0, cp);
            load_w(t + 2, w0);
            cp = load_cp(t + 2 < tile_end ? t + 2 : t);
            if (t + 1 < tile_end) do_tile(t + 1, w1, cp1);
        }
    }
}

// ---------------------------------------------------------------------------------
// MFMA kernel: M <= 16 * MT, K <= WAVES * SEGS * 128 <= 12288
// ---------------------------------------------------------------------------------
// WAVES wavefronts split K: wavefront v owns the 64-byte row segments [v*SEGS, (v+1)*SEGS); lane (l16, g)
// holds bytes [g*16, +16) of each, of weight row l16 of the tile (MFMA "A" side) and of activation rows
// 16*t + l16 of the MT row tiles ("B" side), so it ends up with four consecutive output columns of those rows.
// A weight fragment is expanded once and meets all MT activation fragments: more rows cost matrix instructions
// and registers (MT * SEGS * 4 for the packed activations), not weight traffic.  Nibble -> byte as in the
// GEMM kernels: (w & 0xF0F0F0F0) is the four odd-k nibbles times 16, ((w << 4) & 0xF0F0F0F0) the even ones;
// every product is 256 * a * b and one arithmetic shift recovers the sum.
//
// FUSEQ (one row tile, EPI >= 0): the activations arrive as binary16 and the workgroup quantizes its 16 rows itself,
// 16 / WAVES whole rows per wavefront (so a row's statistics never leave its wavefront), into LDS; the fragments
// then come from there.  Every workgroup repeats that work: it pays while the quantizer's own launch (about 2.6 us
// with the wait between the two) costs more than sixteen rows on a CU's vector units.
template <int WAVES, int SEGS, int EPI, int MT = 1, bool DB = true, bool FUSEQ = false>
__global__ __launch_bounds__(WAVES * 64) void gemm_s4_decode_kernel(DUQ_HEAD_DECL, DecodeParams tail)
{
    const DecodeParams p = with_head(tail, DUQ_HEAD_USE);
    constexpr int MODE = EPI < 0 ? 0 : EPI;
    static_assert(WAVES == 4 || WAVES == 8 || (WAVES == 16 && FUSEQ), "wavefronts per workgroup");
    static_assert(MT >= 1 && MT <= 4, "16-row activation tiles");
    static_assert(!FUSEQ || (MT == 1 && EPI >= 0 && WAVES >= 8 && (WAVES * SEGS) % 4 == 0), "rows quantized in the kernel");
    constexpr int NG = WAVES / 4;             // groups of 256 finishing threads
    constexpr int FT = (MT + NG - 1) / NG;    // row tiles a finishing thread completes
    __shared__ v4i part[2][MT][WAVES][64];
    // FUSEQ: the codes of the 16 rows (a row every XSTRIDE bytes: 16 bytes more than the longest row, so that the 16
    // rows a fragment read touches fall on different banks) and their per-token parameters
    constexpr int RPW = FUSEQ ? 16 / WAVES : 1;        // rows a wavefront quantizes
    constexpr int UPR = FUSEQ ? WAVES * SEGS / 4 : 1;  // 8-element units per lane and row
    constexpr uint32_t XSTRIDE = WAVES * SEGS * 64 + 16;
    __shared__ __attribute__((aligned(16))) uint8_t xs[FUSEQ ? 16 * XSTRIDE : 16];
    __shared__ uint16_t srow[16], zrow[16];
    __shared__ int rsrow[16];
    constexpr bool ASYMQ = FUSEQ && (MODE == 1 || MODE == 3 || MODE == 4 || MODE == 5);
    constexpr bool SHIFTQ = FUSEQ && (MODE == 4 || MODE == 5);

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t l16 = lane & 15u, g = lane >> 4;
    const uint32_t kbytes = p.K >> 1;
    const uint32_t seg0 = wave * SEGS;
    const uint32_t ntiles = (p.N + 15) / 16;
    const uint32_t tile0 = blockIdx.x * p.tiles_per_wg;
    const uint32_t tile_end = min(tile0 + p.tiles_per_wg, ntiles);

    const __amdgpu_buffer_rsrc_t rW = make_rsrc(p.B, p.N * kbytes);  // rows past N read as zero
    uint32_t koff[SEGS];  // byte offset inside a row, or out of range for pieces past K
#pragma unroll
    for (int u = 0; u < SEGS; ++u) {
        const uint32_t off = (seg0 + u) * 64 + g * 16;
        koff[u] = off < kbytes ? off : kOobOffset;
    }
    auto load_tile = [&](uint32_t tile, v4u(&w)[SEGS]) {
        const uint32_t row = tile * 16 + l16;
        const bool rok = tile < tile_end && row < p.N;
#pragma unroll
        for (int u = 0; u < SEGS; ++u)
            w[u] = buf_load16(rW, (rok && koff[u] != kOobOffset) ? row * kbytes + koff[u] : kOobOffset, 0);
    };

    // ---- loads in the order their data is needed (loads return in order): the activation fragments of this
    // wavefront's k range (packed; expanded when used), the first tile's weights, the parameters of the outputs
    // this thread will finish
    v4u xp[MT][SEGS];
    v4u raw[RPW][UPR];
    const uint32_t nunits = p.K >> 3;
    if constexpr (!FUSEQ) {
        const __amdgpu_buffer_rsrc_t rX = make_rsrc(p.A, p.M * kbytes);  // rows past M read as zero
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int u = 0; u < SEGS; ++u)
                xp[t][u] = buf_load16(rX, koff[u] != kOobOffset ? (t * 16 + l16) * kbytes + koff[u] : kOobOffset, 0);
    } else {
        // wavefront v quantizes rows v * RPW ..; lane l owns the 8-element units l, l + 64, ... of each
        const __amdgpu_buffer_rsrc_t rX = make_rsrc(p.X, p.M * p.K * 2);  // rows past M read as zero
#pragma unroll
        for (int r = 0; r < RPW; ++r)
#pragma unroll
            for (int j = 0; j < UPR; ++j) {
                const uint32_t c = lane + j * 64;
                raw[r][j] = buf_load16(rX, c < nunits ? ((wave * RPW + r) * p.K + c * 8) * 2 : kOobOffset, 0);
            }
        // every wavefront requests its activations before any requests weights (requests are served in order)
        __builtin_amdgcn_s_barrier();
    }
    v4u w0[SEGS], w1[DB ? SEGS : 1];
    load_tile(tile0, w0);

    // threads finish one output per row tile they own: element er of MFMA lane src_lane; the 256-thread group
    // fg owns row tiles fg, fg + NG, ...
    const uint32_t src_lane = (tid >> 2) & 63u, er = tid & 3u, fg = tid >> 8;
    const uint32_t my_m = src_lane & 15u, my_c = (src_lane >> 4) * 4 + er;
    const bool bias = p.epi.bias != nullptr;
    const bool finisher = fg < (uint32_t)MT;
    using ColRec = typename EpiRec<MODE>::Col;
    using RowRec = typename EpiRec<MODE>::Row;
    ColRec cp{};
    RowRec rp[FT];
    auto load_cp = [&](uint32_t tile) {
        ColRec c{};
        if (EPI >= 0 && finisher) c = load_col_rt<MODE>(p.epi, min(tile * 16 + my_c, p.N - 1), bias, p.B, kbytes);
        return c;
    };
    cp = load_cp(tile0);
    // (the output pointers arrive in registers)
    const auto c_out = as_global(p.C);
    const auto y_out = as_global(p.y);
#pragma unroll
    for (int f = 0; f < FT; ++f) {
        rp[f] = RowRec{};
        if (EPI >= 0 && finisher && !FUSEQ)
            rp[f] = load_row_rt<MODE>(p.epi, min((fg + f * NG) * 16 + my_m, p.M - 1), p.A, kbytes);
    }

    if constexpr (FUSEQ) {
        // the quantizer's arguments, fetched under the vector loads above (a scalar load issued where its value is
        // first used is waited for on its own)
        const float q_clip = p.clip;
        const int q_qmax = p.qmax;
        uint8_t *const q_out = p.q_out;
        uint16_t *const s_out = p.s_out, *const z_out = p.z_out;
        int32_t *const rs_out = p.rs_out;
        asm volatile("" ::"s"(q_clip), "s"(q_qmax), "s"(q_out), "s"(s_out), "s"(z_out), "s"(rs_out));
        const bool copy_out = blockIdx.x == 0;
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            const uint32_t qrow = wave * RPW + r;
            // units past the row end read as zero: no maximum of |x| changes, a minimum or maximum would
            PkMinMax st;
#pragma unroll
            for (int j = 0; j < UPR; ++j)
                if (!ASYMQ || lane + j * 64 < nunits) st.add8(raw[r][j]);
            uint32_t m16;
            float lo = 0.f, hi = 0.f;
            if (!ASYMQ) {
                m16 = wave_max_u32(st.absmax_bits());
            } else {
                st.wave_reduce();
                m16 = st.absmax_bits();
                lo = st.min_f32();
                hi = st.max_f32();
                if (m16 > 0x7C00u) lo = hi = __builtin_nanf("");  // torch's min / max of a row that holds a NaN
            }
            if (qrow < p.M) {  // rows past M are neither quantized nor used
                RowQuant<ASYMQ> rq;
                rq.init(m16, lo, hi, q_clip, q_qmax);
                int code_sum = 0;
                uint32_t words[UPR];
                quant_in_groups<DUQ_DEC_QUANT_GROUP>(rq, raw[r], words);
#pragma unroll
                for (int j = 0; j < UPR; ++j) {
                    const uint32_t c = lane + j * 64;
                    if (c < nunits) {
                        uint32_t word = words[j];
                        if (SHIFTQ) {
                            const uint32_t pairs = (word & 0x0F0F0F0Fu) + ((word >> 4) & 0x0F0F0F0Fu);
                            code_sum = (int)__builtin_amdgcn_udot4(pairs, 0x01010101u, (uint32_t)code_sum, false);
                            word ^= 0x88888888u;  // u - 8 as a signed nibble
                        }
                        *reinterpret_cast<uint32_t *>(xs + qrow * XSTRIDE + c * 4) = word;
                        if (copy_out && q_out) reinterpret_cast<uint32_t *>(q_out + (uint64_t)qrow * kbytes)[c] = word;
                    }
                }
                if (SHIFTQ) code_sum = wave_sum_i32(code_sum) - 8 * (int)p.K;
                if (lane == 0) {
                    const f16 z = SHIFTQ ? rq.z - (f16)8.0f : rq.z;
                    srow[qrow] = f16_to_bits(rq.s);
                    if (ASYMQ) zrow[qrow] = f16_to_bits(z);
                    if (SHIFTQ) rsrow[qrow] = code_sum;
                    if (copy_out && s_out) s_out[qrow] = f16_to_bits(rq.s);
                    if (ASYMQ && copy_out && z_out) z_out[qrow] = f16_to_bits(z);
                    if (SHIFTQ && copy_out && rs_out) rs_out[qrow] = code_sum;
                }
            }
        }
        __syncthreads();
        // (bytes past the row end, and rows past M, are never written: the weights read as zero there, and a row's
        // codes only reach that row's outputs)
#pragma unroll
        for (int u = 0; u < SEGS; ++u)
            xp[0][u] = koff[u] != kOobOffset ? load16(xs + l16 * XSTRIDE + koff[u]) : v4u{0, 0, 0, 0};
        if (finisher) {
            if constexpr (MODE == 5) {
                const v2u head = *reinterpret_cast<const v2u *>(xs + my_m * XSTRIDE);
                rp[0].xlo = head[0];
                rp[0].xhi = head[1] & 0xFFu;
                rp[0].zx = (uint32_t)rint_i32((float)bits_to_f16(zrow[my_m]));
                rp[0].sx = (float)bits_to_f16(srow[my_m]);
                rp[0].rxl = dual_head_sum(rp[0].xlo, rp[0].xhi);
                rp[0].rxr = (uint32_t)rsrow[my_m] - rp[0].rxl;
            } else {
                rp[0].s = bits_to_f16(srow[my_m]);
                if (ASYMQ) rp[0].z = bits_to_f16(zrow[my_m]);
                if (SHIFTQ) rp[0].rs = rsrow[my_m];
            }
        }
    }

    auto compute_tile = [&](uint32_t tile, const v4u(&w)[SEGS], uint32_t buf) {
        const ColRec cpn = load_cp(tile + 1 < tile_end ? tile + 1 : tile);  // next tile's, under this tile's work
        v4i acc[MT];
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[t] = v4i{0, 0, 0, 0};
#pragma unroll
        for (int u = 0; u < SEGS; ++u) {
            v4u we, wo;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                we[q] = (w[u][q] << 4) & kNibbleMaskD;
                wo[q] = w[u][q] & kNibbleMaskD;
            }
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                v4u xe, xo, xv = xp[t][u];
                // many fragments: keep their expansion here (hoisted out of the tile loop it would double the
                // registers they take)
                if (MT * SEGS > 16) asm volatile("" : "+v"(xv));
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    xe[q] = (xv[q] << 4) & kNibbleMaskD;
                    xo[q] = xv[q] & kNibbleMaskD;
                }
                acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(v4i, we), __builtin_bit_cast(v4i, xe), acc[t], 0, 0, 0);
                acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(v4i, wo), __builtin_bit_cast(v4i, xo), acc[t], 0, 0, 0);
            }
        }
#pragma unroll
        for (int t = 0; t < MT; ++t) part[buf][t][wave][lane] = acc[t];
        __syncthreads();
#pragma unroll
        for (int f = 0; f < FT; ++f) {
            const uint32_t t = fg + f * NG;
            if (t < (uint32_t)MT) {
                int sum = 0;
#pragma unroll
                for (int w2 = 0; w2 < WAVES; ++w2) sum += part[buf][t][w2][src_lane][er];
                sum >>= 8;
                const uint32_t m = t * 16 + my_m, n = tile * 16 + my_c;
                if (m < p.M && n < p.N) {
                    if (EPI < 0)
                        c_out[(uint64_t)m * p.N + n] = sum;
                    else
                        y_out[(uint64_t)m * p.N + n] = dequant_rt<MODE>(sum, rp[f], cp, bias);
                }
            }
        }
        cp = cpn;
    };

    // two register sets alternate so that one tile's loads are in flight during the other's MFMAs; the
    // partial-sum buffers alternate too: one barrier per tile.  (DB = false: one set, for the long rows whose
    // fragments leave no room for a second; their layers have at most 256 column tiles, one per workgroup.)
    if constexpr (DB) {
        for (uint32_t t = tile0; t < tile_end; t += 2) {
            load_tile(t + 1, w1);
            compute_tile(t, w0, 0);
            load_tile(t + 2, w0);
            if (t + 1 < tile_end) compute_tile(t + 1, w1, 1);
        }
    } else {
        for (uint32_t t = tile0; t < tile_end; ++t) {
            if (t != tile0) load_tile(t, w0);
            compute_tile(t, w0, (t - tile0) & 1u);
        }
    }
}

// ---------------------------------------------------------------------------------
// dispatch
// ---------------------------------------------------------------------------------
// Every dispatcher below returns whether it launched a kernel: a shape or mode that no instantiated template
// covers launches nothing, and the entry points turn that into an error instead of returning success with the
// output unwritten.
template <int MR, int XS, bool FUSEQ>
bool launch_rows_mode(DecodeParams &p, int epi, hipStream_t stream)
{
    const uint32_t ntiles = (p.N + 4 * DUQ_DEC_R - 1) / (4 * DUQ_DEC_R);  // 16 weight rows per tile
    // One tile per workgroup.  Four rows quantized in the kernel, more than 256 tiles: every workgroup quantizes
    // the rows again, so one round of at most 256 workgroups of eight wavefronts with several tiles each when two
    // register sets of weights fit (rows of at most 8192 elements; measured at K = 4096: N = 6144 5.76 against
    // 6.21 us, N = 11008 7.18 against 7.73).  On pre-quantized rows, or with one or two rows, several tiles per
    // workgroup measured 3-15 % slower than one (four wavefronts per CU keep too few loads in flight): not used
    // there.
    constexpr bool kCanMulti = FUSEQ && MR >= 4 && XS <= (MR == 4 ? 4 : 2);
    const bool multi = kCanMulti && ntiles > 256;
    p.tiles_per_wg = multi ? (ntiles + 255) / 256 : 1;
    const dim3 grid((ntiles + p.tiles_per_wg - 1) / p.tiles_per_wg);
    // wavefronts per workgroup: four, or with three or more rows to quantize WQ (DUQ_DEC_FUSEQ_WAVES above)
    constexpr int WQ = !FUSEQ || MR == 1 ? 4
                       : MR == 2         ? DUQ_DEC_FUSEQ_WAVES_M2
                       : MR == 8         ? (XS >= 4 ? DUQ_DEC_FUSEQ_WAVES_M8L : DUQ_DEC_FUSEQ_WAVES)
                                         : (XS >= 4 ? DUQ_DEC_FUSEQ_WAVES_M4L : DUQ_DEC_FUSEQ_WAVES_M4);
    constexpr int WMULTI = DUQ_DEC_FUSEQ_WAVES;
    bool launched = false;
#define DUQ_ROWS(E)                                                                                              \
    if (multi) {                                                                                                 \
        if constexpr (kCanMulti) {                                                                               \
            DUQ_LAUNCH_HEAD((gemv_s4_rows_kernel<MR, XS, FUSEQ, E, WMULTI, true>), grid, dim3(WMULTI * 64), 0, stream, p); \
            launched = true;                                                                                     \
        }                                                                                                        \
    } else {                                                                                                     \
        DUQ_LAUNCH_HEAD((gemv_s4_rows_kernel<MR, XS, FUSEQ, E, WQ>), grid, dim3(WQ * 64), 0, stream, p);              \
        launched = true;                                                                                         \
    }
    switch (epi) {
    case 0: DUQ_ROWS(0) break;
    case 1: DUQ_ROWS(1) break;
    case 2: DUQ_ROWS(2) break;
    case 3: DUQ_ROWS(3) break;
    case 4: DUQ_ROWS(4) break;
    case 5: DUQ_ROWS(5) break;
    default:
        if constexpr (!FUSEQ) {
            if (epi == -1) { DUQ_ROWS(-1) }
        }
    }
#undef DUQ_ROWS
    return launched;
}

template <int MR, bool FUSEQ>
bool launch_rows_xs(DecodeParams &p, int epi, hipStream_t stream)
{
    const uint32_t kbytes = p.K / 2;
    if (kbytes <= 2048) return launch_rows_mode<MR, 2, FUSEQ>(p, epi, stream);
    if (kbytes <= 4096) return launch_rows_mode<MR, 4, FUSEQ>(p, epi, stream);
    if constexpr (MR <= 4) {  // (eight rows: up to 8192 elements, decode_fp16in_one_launch)
        if (kbytes <= 6144) return launch_rows_mode<MR, 6, FUSEQ>(p, epi, stream);
        if (kbytes <= 8192) return launch_rows_mode<MR, 8, FUSEQ>(p, epi, stream);
    }
    return false;
}

template <int WAVES, int SEGS, int MT = 1, bool DB = true, bool FUSEQ = false>
bool launch_mfma_mode(const DecodeParams &p, int epi, hipStream_t stream)
{
    const uint32_t ntiles = (p.N + 15) / 16;
    const dim3 grid((ntiles + p.tiles_per_wg - 1) / p.tiles_per_wg);
#define DUQ_DEC(E) \
    DUQ_LAUNCH_HEAD((gemm_s4_decode_kernel<WAVES, SEGS, E, MT, DB, FUSEQ>), grid, dim3(WAVES * 64), 0, stream, p)
    switch (epi) {
    case -1:
        if constexpr (FUSEQ) return false;
        else DUQ_DEC(-1);
        break;
    case 0: DUQ_DEC(0); break;
    case 1: DUQ_DEC(1); break;
    case 2: DUQ_DEC(2); break;
    case 3: DUQ_DEC(3); break;
    case 4: DUQ_DEC(4); break;
    case 5: DUQ_DEC(5); break;
    default: return false;
    }
#undef DUQ_DEC
    return true;
}

template <bool FUSEQ>
bool launch_decode_any(DecodeParams &p, int epi, hipStream_t stream)
{
    const uint32_t kbytes = p.K / 2;
    if (decode_uses_rows_kernel(p.M)) {
        if (p.M == 1) return launch_rows_xs<1, FUSEQ>(p, epi, stream);
        if (p.M == 2) return launch_rows_xs<2, FUSEQ>(p, epi, stream);
        return launch_rows_xs<4, FUSEQ>(p, epi, stream);
    }
    if constexpr (FUSEQ) {
#ifndef DUQ_DEC_M8_MFMA
        if (p.M <= 8) return launch_rows_xs<8, true>(p, epi, stream);  // 5..8 rows
#endif
        if (p.M > 16 || kbytes > 2048) return false;
        // 9..16 rows: the MFMA kernel, rows quantized by every workgroup
        constexpr int W = DUQ_DEC_MFMA_FUSEQ_WAVES;
        p.tiles_per_wg = decode_tiles_per_workgroup((p.N + 15) / 16);
        if (kbytes <= 1024) return launch_mfma_mode<W, 16 / W, 1, true, true>(p, epi, stream);
        return launch_mfma_mode<W, 32 / W, 1, true, true>(p, epi, stream);
    } else {
        const uint32_t ntiles = (p.N + 15) / 16;
        p.tiles_per_wg = decode_tiles_per_workgroup(ntiles);
        constexpr int W = DUQ_DEC_WAVES, S = 32 / W;  // 64-byte segments per wavefront for 2 KB of a row
        const uint32_t mt = (p.M + 15) / 16;
        // rows of up to 4096 / 8192 / 12288 elements: S, 2 S, 12 segments per wavefront; the row tiles whose
        // fragments fit in registers next to two sets of weights (what select_gemm_kernel sends here)
        if (mt > 4 || kbytes > 6144) return false;
        if (kbytes <= 2048) {
            if (mt == 1) return launch_mfma_mode<W, S, 1>(p, epi, stream);
            if (mt == 2) return launch_mfma_mode<W, S, 2>(p, epi, stream);
            if (mt == 3) return launch_mfma_mode<W, S, 3>(p, epi, stream);
            return launch_mfma_mode<W, S, 4>(p, epi, stream);
        }
        if (kbytes <= 4096) {
            if (mt == 1) return launch_mfma_mode<W, 2 * S, 1>(p, epi, stream);
            if (mt == 2) return launch_mfma_mode<W, 2 * S, 2>(p, epi, stream);
            if (mt == 3) return launch_mfma_mode<W, 2 * S, 3>(p, epi, stream);
            return launch_mfma_mode<W, 2 * S, 4>(p, epi, stream);
        }
        if (mt == 1) return launch_mfma_mode<8, 12, 1>(p, epi, stream);
        if (mt == 2) return launch_mfma_mode<8, 12, 2, false>(p, epi, stream);
        if (mt == 3) return launch_mfma_mode<8, 12, 3, false>(p, epi, stream);
        return false;
    }
}

}  // namespace

// Measurement aid: the rows kernel's access pattern without its arithmetic (every lane requests 8 x 16 bytes up
// front, a load instruction covers 1 KB, one workgroup per 32 KB) over `bytes` of memory, nothing stored.  What
// this takes for N * K / 2 bytes is the floor of a decode launch of that size on the part.
__global__ __launch_bounds__(256) void probe_read_kernel(const v4u *src, uint32_t nvec, uint32_t *sink)
{
    const uint32_t gw = (blockIdx.x * 256 + threadIdx.x) >> 6, lane = threadIdx.x & 63u;
    const __amdgpu_buffer_rsrc_t r = make_rsrc(src, nvec * 16);
    v4u v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t idx = gw * 512 + i * 64 + lane;
        v[i] = __builtin_bit_cast(
            v4u, __builtin_amdgcn_raw_buffer_load_b128(r, (int)(idx < nvec ? idx * 16 : kOobOffset), 0, DUQ_DEC_WLOAD_AUX));
    }
    uint32_t x = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) x ^= (v[i][0] ^ v[i][1]) ^ (v[i][2] ^ v[i][3]);
    if (x == 0x9E3779B9u && sink) sink[gw & 63u] = x;  // keeps the loads alive; practically never taken
}

int launch_probe_read(const void *src, uint64_t bytes, uint32_t *sink, hipStream_t stream)
{
    const uint32_t nvec = (uint32_t)(bytes / 16);
    if (nvec == 0) return 0;
    const uint32_t waves = (nvec + 511) / 512;
    hipLaunchKernelGGL(probe_read_kernel, dim3((waves + 3) / 4), dim3(256), 0, stream, static_cast<const v4u *>(src), nvec,
                       sink);
    return (int)hipGetLastError();
}

int launch_decode_s4(const uint8_t *A, const uint8_t *B, uint32_t M, uint32_t N, uint32_t K, int32_t *out_acc,
                     const Epilogue *epi, uint16_t *y, hipStream_t stream)
{
    DecodeParams p{};
    p.A = A;
    p.B = B;
    p.M = M;
    p.N = N;
    p.K = K;
    p.C = out_acc;
    p.y = y;
    if (epi) p.epi = *epi;
    if (!launch_decode_any<false>(p, out_acc ? -1 : epi->mode, stream)) return (int)hipErrorInvalidValue;
    return (int)hipGetLastError();
}

int launch_decode_fp16in(const uint16_t *x, float clip, int qmax, const uint8_t *B, uint32_t M, uint32_t N, uint32_t K,
                         const Epilogue &epi, uint16_t *y, uint8_t *q_out, uint16_t *s_out, uint16_t *z_out,
                         int32_t *rs_out, hipStream_t stream)
{
    DecodeParams p{};
    p.X = x;
    p.B = B;
    p.M = M;
    p.N = N;
    p.K = K;
    p.y = y;
    p.epi = epi;
    p.clip = clip;
    p.qmax = qmax;
    p.q_out = q_out;
    p.s_out = s_out;
    p.z_out = z_out;
    p.rs_out = rs_out;
    if (!launch_decode_any<true>(p, epi.mode, stream)) return (int)hipErrorInvalidValue;
    return (int)hipGetLastError();
}

}  // namespace duq
