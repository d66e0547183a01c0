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
inline bool decode_uses_rows_kernel(uint32_t M) { return M <= 4; }
// MFMA decode kernel: one round of at most 256 workgroups, each with its share of the 16-column tiles.  The
// activations enter a CU once, and a workgroup has two tiles' weights in flight whatever their number; measured
// against one tile per workgroup (16 rows, K = 4096): N = 4800 4.96 against 6.54 us, N = 8192 5.67 against 6.89,
// N = 11008 7.05 against 8.78; 64 rows, N = 11008: 10.95 against 15.7.
inline uint32_t decode_tiles_per_workgroup(uint32_t ntiles) { return (ntiles + 255) / 256; }
// quantize + GEMM + dequant from binary16 activations in one launch: shapes of the rows kernel, and 5..8 rows
// of at most 4096 elements, or 8192 on at most 4096 columns (the rows kernel with eight rows, one wavefront
// quantizing each; measured against quantizer + MFMA decode kernel at 8 rows: N = K = 4096 6.3 against 7.2 us,
// N = 11008 8.5 against 9.8, K = 2048 4.9 against 6.4, N = K = 8192 16.9 against 13.5); from two rows on only up to
// 16384 output columns (every workgroup quantizes the rows again: measured slower than two launches beyond)
inline bool decode_fp16in_one_launch(uint32_t M, uint32_t N, uint32_t K)
{
    const int kernel = select_gemm_kernel(M, N, K);
    if (kernel == kKernelDecodeRows) return M == 1 || N <= 16384;
    return M <= 8 && N <= 16384 && (K <= 4096 || (K <= 8192 && N <= 4096)) && kernel == kKernelDecodeMfma;
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
