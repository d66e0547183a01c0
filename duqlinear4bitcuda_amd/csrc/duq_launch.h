// Host-side launchers implemented by the .hip files; the extern "C" layer in
// duq_abi.hip validates arguments and forwards here.  All return a hipError_t as int.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <algorithm>

namespace duq {

int launch_sym_quant(const uint16_t *x, const uint16_t *scale, uint32_t rows, uint32_t colsSrc, uint32_t colsDst,
                     int qmax, uint8_t *q, hipStream_t stream);
int launch_sym_dual_quant(const uint16_t *x, const uint16_t *s1, const uint16_t *s2, uint32_t rows,
                          uint32_t colsSrc, uint32_t colsDst, int qmax, uint8_t *q, hipStream_t stream);
int launch_asym_quant(const uint16_t *x, const uint16_t *scale, const uint16_t *zeros, uint32_t rows,
                      uint32_t colsSrc, uint32_t colsDst, uint8_t *q, hipStream_t stream);
int launch_asym_dual_quant(const uint16_t *x, const uint16_t *s1, const uint16_t *z1, const uint16_t *s2,
                           const uint16_t *z2, uint32_t rows, uint32_t colsSrc, uint32_t colsDst, uint8_t *q,
                           hipStream_t stream);
// bf6 != nullptr (cols % 128 == 0): also write the E3M2 shadow of the codes; q may then be nullptr.
int launch_quantize_rows_sym(const uint16_t *x, uint32_t rows, uint32_t cols, float clip, int qmax, uint8_t *q,
                             uint16_t *scale, uint8_t *bf6, hipStream_t stream);
// rowsum == nullptr: unsigned codes and zero points as the reference stores them; otherwise the
// signed-shifted form (code - 8, zero - 8) plus the per-row sum of the shifted codes.
int launch_quantize_rows_asym(const uint16_t *x, uint32_t rows, uint32_t cols, uint8_t *q, uint16_t *scale,
                              uint16_t *zeros, int32_t *rowsum, uint8_t *bf6, hipStream_t stream);

// Epilogue description shared by the stand-alone dequant kernels and the fused GEMM.
// mode: 0 sym, 1 asym, 2 sym-dual, 3 asym-dual, 4 asym with row-sum zero-point correction, 5 the same for the
// dual-uniform layer (fused GEMM only, shapes of gemm_fuses_dual_rowsum) (DUQ_EPI_* of the public header).
struct Epilogue {
    int mode;
    const uint16_t *s_row;   // [rows]
    const uint16_t *z_row;   // [rows]  asym modes
    const uint16_t *s_col_1; // [cols]
    const uint16_t *z_col_1; // [cols]  asym modes
    const uint16_t *s_col_2; // [cols]  dual modes
    const uint16_t *z_col_2; // [cols]  asym-dual
    const uint16_t *bias;    // [cols] or nullptr
    const int32_t *rs_row;   // [rows]  mode 4: sum over k of the row's shifted codes
    const int32_t *rs_col;   // [cols]  mode 4: sum over k of the column's shifted codes minus K * zero (mode 5: of
                             //         input columns 0..9)
    const int32_t *rs_col_2; // [cols]  mode 5: the same over the other input columns
};

int launch_dequant(const int32_t *acc, const Epilogue &epi, uint32_t rows, uint32_t cols, uint16_t *y,
                   hipStream_t stream);
// the same over `batches` accumulator matrices [batches, rows, cols] in one launch, every batch entry with its
// own per-row [batches, rows] and per-column [batches, cols] parameters.  batches <= 65535.
int launch_dequant_batched(const int32_t *acc, const Epilogue &epi, uint32_t batches, uint32_t rows, uint32_t cols,
                           uint16_t *y, hipStream_t stream);

// Row-sum epilogue of the dual-uniform layer on int32 accumulators (definition: include/duq_hip.h,
// duq_asym_dual_rowsum_dequant_host).  xq / w are the packed operands of the GEMM that made `acc`: the kernel reads
// the first eight bytes of every row of both (the codes of input columns 0..9).
struct DualRowsumParams {
    const int32_t *acc;      // [rows, cols]
    const uint8_t *xq;       // [rows, kbytes]
    const uint8_t *w;        // [cols, kbytes]
    uint32_t kbytes;
    const uint16_t *s_row, *z_row;   // [rows]
    const int32_t *rs_row;           // [rows]
    const uint16_t *s_col_1, *z_col_1, *s_col_2, *z_col_2;  // [cols]
    const int32_t *adj_col_1, *adj_col_2;                   // [cols]
    const uint16_t *bias;            // [cols] or nullptr
    uint32_t rows, cols;
    uint16_t *y;             // [rows, cols]
};
int launch_dual_rowsum_dequant(const DualRowsumParams &p, hipStream_t stream);

// Kernel families of the int4 GEMM and the host-side rule that picks one (select_gemm_kernel: host arithmetic
// only, exported as duq_gemm_kernel_for so that the rule can be tested without a GPU).
enum GemmKernelId {
    kKernelDecodeRows = 1,  // duq_decode.hip, v_dot8_i32_i4, M <= 4
    kKernelDecodeMfma = 2,  // duq_decode.hip, MFMA, 5 <= M <= 16 (K <= 12288), 17 <= M <= 64 (K <= 8192; 48 rows: 12288)
    kKernelDot = 3,         // duq_gemm.hip, M <= 4 with rows longer than 16384 elements
    kKernelRing = 4,        // duq_gemm.hip, 17 <= M <= 256 on narrow problems the decode kernel does not take
    kKernelSkinny = 5,      // duq_gemm.hip, 9 <= M <= 16 with 1536 or more column tiles, K <= 4096
    kKernelStream = 6,      // duq_gemm.hip, prefill
    kKernelTile = 7,        // duq_gemm.hip, everything else (per-tile 64-bit bases: any tensor size)
};
int select_gemm_kernel(uint32_t M, uint32_t N, uint32_t K);
// Shapes whose GEMM can apply the dual-uniform row-sum epilogue itself (mode 5): those of the decode kernels, and those
// of the stream kernel with rows longer than 256 elements and N % 8 == 0 (its staged stores); the others run the GEMM
// into int32 and launch_dual_rowsum_dequant.
inline bool gemm_fuses_dual_rowsum(uint32_t M, uint32_t N, uint32_t K)
{
    const int kernel = select_gemm_kernel(M, N, K);
    if (kernel == kKernelDecodeRows || kernel == kKernelDecodeMfma) return true;
    return kernel == kKernelStream && K > 256 && N % 8 == 0;
}
// Tile of the stream kernel for a problem select_gemm_kernel gives to it (rows 0: none, the tile kernels run).
// Whole rounds of 256 workgroups (one per CU) cost about nchunks * c + f microseconds each, c (per 256 k) and f
// measured per tile shape; the cheapest wins.  The L2 -> CU path bounds these tiles, so what counts is operand rows
// per output: a 64 x 128 tile has the outputs of a 32 x 256 one with a third less operand bytes into the CU (192 rows
// of K / 2 bytes against 288): 512 x 4096 x 4096 13.1 against 19.8 us, 512 x 4096 x 11008 (K) 34.1 against 52; a
// 128 x 128 tile those of a 64 x 256 one with a fifth less (256 against 320): 1024 x 4096 x 4096 21.5 against 26.1 us
// on one box, 768 rows 18.9 against 22.4, 1024 x 4096 x 11008 (K) 50.5 against 58.5.  A round of 256 x 256 tiles
// (gemm_s4_stream256_kernel; not with the dual-uniform row-sum epilogue, `mode5`) costs 1.91 rounds of 128 x 256
// ones for twice the outputs, measured (us, 256-row against 128-row tiles): 4096 x 4096 x 4096 56.5 / 58.9,
// 4096 x 11008 x 4096 149 / 160, 2048 x 22016 x 4096 150 / 160, 4096 x 28672 x 8192 668 / 707,
// 4096 x 8192 x 28672 (K) 634 / 667; and 4000 x 8200 x 4160, three ragged rounds against five: 160 / 145.
struct StreamTile {
    uint32_t rows, cols;
};
inline StreamTile select_stream_tile(uint32_t M, uint32_t N, uint32_t K, uint32_t batch, bool mode5)
{
    auto tiles = [&](uint32_t bm, uint32_t bn) { return ((M + bm - 1) / bm) * ((N + bn - 1) / bn) * batch; };
    const float nch = (float)((K + 255) / 256);
    const uint32_t tm[5] = {4, 2, 1, 2, 4};
    const bool hw[5] = {false, false, false, true, true};
    const float c_us[5] = {1.5f, 1.0f, 0.8f, 0.78f, 0.9f}, f_us[5] = {9.f, 7.f, 6.f, 1.f, 4.5f};
    StreamTile best{0, 0};
    float best_cost = 0.f;
    for (int k = 0; k < 5; ++k) {
        const uint32_t t = tiles(32u * tm[k], hw[k] ? 128 : 256);
        const float cost = (float)((t + 255) / 256) * (nch * c_us[k] + f_us[k]);
        if (best.rows == 0 || cost < best_cost) {
            best_cost = cost;
            best = StreamTile{32u * tm[k], hw[k] ? 128u : 256u};
        }
    }
    const uint32_t t256 = tiles(256, 256);
    if (!mode5 && K > 256 && t256 >= 256 && 1.91f * (float)((t256 + 255) / 256) * (nch * c_us[0] + f_us[0]) < best_cost)
        best = StreamTile{256, 256};
    return best;
}
inline bool decode_uses_rows_kernel(uint32_t M) { return M <= 4; }
// MFMA decode kernel: one round of at most 256 workgroups, each with its share of the 16-column tiles.  The
// activations enter a CU once, and a workgroup has two tiles' weights in flight whatever their number; measured
// against one tile per workgroup (16 rows, K = 4096): N = 4800 4.96 against 6.54 us, N = 8192 5.67 against 6.89,
// N = 11008 7.05 against 8.78; 64 rows, N = 11008: 10.95 against 15.7.
inline uint32_t decode_tiles_per_workgroup(uint32_t ntiles) { return (ntiles + 255) / 256; }
// quantize + GEMM + dequant from binary16 activations in one launch: shapes of the rows kernel, and 5..8 rows
// of at most 4096 elements, or 8192 on at most 4096 columns (the rows kernel with eight rows, one wavefront
// quantizing each; measured against quantizer + MFMA decode kernel at 8 rows: N = K = 4096 4.7 against 6.5 us,
// N = 11008 7.2 against 9.3, N = 28672 13.0 against 16.0, N = 65536 K = 2048 18.7 against 21.5; K = 8192: N = 8192
// 15.3 against 13.0, N = 11008 21.0 against 15.0).  Two to four rows longer than 8192 elements only up to 16384
// output columns: every workgroup quantizes the rows again (4 rows: N = 28672 K = 8192 20.5 - 21.9 against 23.4 us,
// N = 32000 K = 4096 12.6 against 14.1, N = 128256 K = 4096 41.3 against 42.4, but N = 20000 K = 16384 45.2 against
// 36.3).
// 9..16 rows: the MFMA kernel with sixteen wavefronts, one quantizing each row, while the rows together hold at most
// 32768 elements, 40960 on at most 4096 columns (measured against two launches, N = 4096: 16 rows of 2048 4.9 against
// 6.0 us, of 1024 4.1 against 5.3, 10 of 3072 5.9 against 6.3, 9 of 4096 6.2 against 6.5; 16 of 3072 6.45 either way,
// 16 of 4096 7.2 against 6.55: each CU then spends 2 us of vector work and 0.85 us of fetching on the rows.  16 rows
// of 2048: N = 8192 5.9 against 6.6, N = 16384 8.4 against 8.9; 10 of 4096 on N = 11008 9.3 either way, 13 of 3072
// on N = 11008 9.0 against 8.6).
inline bool decode_fp16in_one_launch(uint32_t M, uint32_t N, uint32_t K)
{
    const int kernel = select_gemm_kernel(M, N, K);
    if (kernel == kKernelDecodeRows) return M == 1 || N <= 16384 || K <= 8192;
#ifndef DUQ_DEC_FUSEQ16_ELEMS
#define DUQ_DEC_FUSEQ16_ELEMS 32768u
#define DUQ_DEC_FUSEQ16_ELEMS_NARROW 40960u
#endif
    if (M > 8)
        return M <= 16 && K <= 4096 && M * K <= (N <= 4096 ? DUQ_DEC_FUSEQ16_ELEMS_NARROW : DUQ_DEC_FUSEQ16_ELEMS) && N <= 16384 &&
               kernel == kKernelDecodeMfma;
    return M <= 8 && (K <= 4096 || (K <= 8192 && N <= 4096)) && kernel == kKernelDecodeMfma;
}
// decode kernels (duq_decode.hip); the shape must be one select_gemm_kernel gives to them
int launch_decode_s4(const uint8_t *A, const uint8_t *B, uint32_t M, uint32_t N, uint32_t K, int32_t *out_acc,
                     const Epilogue *epi, uint16_t *y, hipStream_t stream);
// the same with binary16 activations in: the per-token quantizer runs inside the launch, SymQuantizer for the
// symmetric epilogues (scale = h(h(max|x| / 7) * clip), codes clamp(rint(h(x / scale)), -8, qmax)), AsymQuantizer for
// modes 1 and 3 (unsigned codes, as the reference stores them) and its signed-shifted form for modes 4 and 5 (codes and
// zero points minus 8, plus the per-token sums of the shifted codes); epi.s_row / z_row / rs_row are ignored.
// q_out / s_out / z_out / rs_out (optional) receive the codes, scales, zero points and sums.  Shapes of
// decode_fp16in_one_launch only.
int launch_decode_fp16in(const uint16_t *x, float clip, int qmax, const uint8_t *B, uint32_t M, uint32_t N, uint32_t K,
                         const Epilogue &epi, uint16_t *y, uint8_t *q_out, uint16_t *s_out, uint16_t *z_out,
                         int32_t *rs_out, hipStream_t stream);

// measurement aid: read `bytes` (< 4 GiB) with the decode kernels' access pattern and discard them
int launch_probe_read(const void *src, uint64_t bytes, uint32_t *sink, hipStream_t stream);

// GEMM: out_acc != nullptr -> int32 accumulators [M,N]; else fused epilogue into y.
int launch_gemm_s4(const uint8_t *A, const uint8_t *B, uint32_t M, uint32_t N, uint32_t K, int32_t *out_acc,
                   const Epilogue *epi, uint16_t *y, hipStream_t stream);
// `batch` problems of one shape in one launch: A [batch, M, K/2], B [batch, N, K/2], out [batch, M, N], the
// epilogue's per-row arrays [batch, M] and per-column arrays [batch, N], all contiguous.  batch <= 65535.
int launch_gemm_s4_batched(const uint8_t *A, const uint8_t *B, uint32_t M, uint32_t N, uint32_t K, uint32_t batch,
                           int32_t *out_acc, const Epilogue *epi, uint16_t *y, hipStream_t stream);


// 6-bit float (E3M2) shadows of packed-int4 tensors and the GEMM that multiplies them
// (duq_bf6.hip).  K % 128 == 0, N % 16 == 0.
int launch_weight_shadow_bf6(const uint8_t *w, uint32_t N, uint32_t K, uint8_t *out, hipStream_t stream);
int launch_activation_shadow_bf6(const uint8_t *q, uint32_t M, uint32_t K, uint8_t *out, hipStream_t stream);
// epi.mode 5 (row-sum epilogue of the dual-uniform layer) also needs the packed-int4 operands the shadows were made
// from, xq [M, K/2] and wq [N, K/2]: the first eight bytes of every row are read.
int launch_gemm_bf6(const uint8_t *X, const uint8_t *W, uint32_t M, uint32_t N, uint32_t K, const Epilogue &epi,
                    uint16_t *y, hipStream_t stream, const uint8_t *xq = nullptr, const uint8_t *wq = nullptr);

// 8-bit asymmetric layer (duq_int8.hip): float32 activations, int8 codes, int32 accumulators, float32 results.
int launch_asym_quant8(const float *x, const float *scale, const float *zeros, uint32_t rows, uint32_t cols, int8_t *q,
                       hipStream_t stream);
int launch_quantize_rows_asym8(const float *x, uint32_t rows, uint32_t cols, int8_t *q, float *scale, float *zeros,
                               hipStream_t stream);
int launch_dequant_hprec(const int32_t *acc, const float *s_row, const float *z_row, const float *s_col,
                         const float *z_col, const float *bias, uint32_t rows, uint32_t cols, float *x,
                         hipStream_t stream);
// C != nullptr -> int32 accumulators [M,N]; else the float32 dequant (+ bias) fused into y.
// b_tiled: B is the output of launch_weight_tile8 (fused form only).
int launch_gemm_s8(const int8_t *A, const int8_t *B, bool b_tiled, uint32_t M, uint32_t N, uint32_t K, int32_t *C,
                   const float *s_row, const float *z_row, const float *s_col, const float *z_col, const float *bias,
                   float *y, hipStream_t stream);
int launch_weight_tile8(const int8_t *w, uint32_t N, uint32_t K, int8_t *out, hipStream_t stream);

}  // namespace duq
