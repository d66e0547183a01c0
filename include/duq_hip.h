/*
 * duq_hip.h - C ABI of libduq_hip.so, the MI355X (gfx950) implementation of the
 * Linear4bit forward path: per-token int4 quantize -> s4 x s4 GEMM (int32) -> fp16
 * dequant.
 *
 * Every entry point replaces one raw-pointer host launcher of the reference (cited per
 * function, paths relative to the reference checkout) and keeps its argument order and
 * meaning, with three changes that hold throughout:
 *   - binary16 values travel as `duq_half` (uint16_t bit patterns) so the header needs
 *     no GPU toolkit;
 *   - a trailing `duq_stream_t` (a hipStream_t, NULL = the null stream) is added: the
 *     reference always launches on the legacy default stream;
 *   - the functions return a status instead of void: 0 on success, a negative DUQ_E_*
 *     code for a rejected argument, or a positive hipError_t from the launch.  They
 *     never exit, abort or throw.
 *
 * All pointers are DEVICE pointers on the current HIP device; inputs are borrowed,
 * outputs are caller-allocated, the library allocates no memory and keeps no global state
 * (re-entrant); the one exception is duq_quantize_linear4bit_forward_static and its static
 * device array (and duq_static_scratch_init, which belongs to it).  No call synchronises the host.
 *
 * Packed int4 layout everywhere: element i of a row is in byte i/2, low nibble first
 * (include/int4.h:86-98).
 */
#ifndef DUQ_HIP_H
#define DUQ_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef uint16_t duq_half;   /* IEEE binary16 bit pattern */
typedef void *duq_stream_t;  /* hipStream_t */

/* status codes (negative = argument rejected before any launch) */
#define DUQ_OK 0
#define DUQ_E_NULL (-1)      /* a required pointer is NULL */
#define DUQ_E_SHAPE (-2)     /* a dimension is inconsistent (e.g. colsDst != ceil(colsSrc/2)) */
#define DUQ_E_KALIGN (-3)    /* GEMM K is not a multiple of 64 (qlinear4bit/tools/tensor_utils.py:52) */
#define DUQ_E_MODE (-4)      /* unknown epilogue mode / unsupported qmax */
#define DUQ_E_ALIGN (-5)     /* a pointer misses the alignment the entry point documents */
#define DUQ_E_TOO_LARGE (-6) /* a dimension exceeds what the kernels index with 32 bits: K > 131008, N > 2^22, M > 2^24 */
#define DUQ_E_SCRATCH (-7)   /* the input does not fit a slot of the static scratch buffer of the entry point that allocates nothing, or the slot does not exist */
#define DUQ_E_DEVICE (-8)    /* the stream belongs to another device than the current one */
#define DUQ_E_CAPTURE (-9)   /* a call that must query the runtime was made on a stream under capture */

/* symmetric clamp used by the device quantizer of the reference: qmax_sym evaluates to 6
 * (include/common.h:53-54).  7 is the bound of the Python fake-quant path
 * (qlinear4bit/tools/quantization.py:29-32). */
#define DUQ_QMAX_SYM_DEVICE 6
#define DUQ_QMAX_SYM_FAKEQUANT 7
#define DUQ_QUANT_COL_K 10   /* include/quant.h:5 */

/* epilogue selectors for duq_linear4bit_forward */
#define DUQ_EPI_SYM 0        /* src/kernels/quant.cu:64-81   */
#define DUQ_EPI_ASYM 1       /* src/kernels/quant.cu:149-169 */
#define DUQ_EPI_SYM_DUAL 2   /* src/kernels/quant2.cu:62-83  */
#define DUQ_EPI_ASYM_DUAL 3  /* src/kernels/quant2.cu:158-186 */
#define DUQ_EPI_ASYM_ROWSUM 4 /* exact zero-point correction with row sums; not in the reference */
#define DUQ_EPI_ASYM_DUAL_ROWSUM 5 /* the same for the dual-uniform layer (duq_linear4bit_forward_dual_rowsum only) */

/* ---- library info ------------------------------------------------------------------ */

/* ABI version of this header (bumped on incompatible change). */
int duq_abi_version(void);
/* Text for a status code returned by any function below (static storage). */
const char *duq_status_string(int status);
/* QUANT_COL_K; replaces get_dual_quant_col_k (src/export/bindings.cpp:471-473). */
int duq_get_dual_quant_col_k(void);

/* ---- per-token quantizers with caller-supplied scales ------------------------------- */

/* Replaces sym_quant_host (include/quant.h:9-16, src/kernels/quant.cu:48-61).
 * q[r, j] packs clamp(rint(x[r,2j]/scale[r]), -8, 6) and the same for 2j+1; the division
 * is the binary16 quotient, rounding is to nearest even.  colsDst must be
 * ceil(colsSrc/2); an odd colsSrc leaves the last high nibble 0. */
int duq_sym_quant_host(const duq_half *x, const duq_half *scale, uint32_t rows, uint32_t colsSrc,
                       uint32_t colsDst, uint8_t *q, duq_stream_t stream);
/* Same with an explicit upper clamp (6 or 7). */
int duq_sym_quant_host_qmax(const duq_half *x, const duq_half *scale, uint32_t rows, uint32_t colsSrc,
                            uint32_t colsDst, int32_t qmax, uint8_t *q, duq_stream_t stream);

/* Replaces sym_dual_quant_host (include/quant.h:29-37, src/kernels/quant2.cu:47-60):
 * columns < 10 use scale_1[r], the others scale_2[r]. */
int duq_sym_dual_quant_host(const duq_half *x, const duq_half *scale_1, const duq_half *scale_2,
                            uint32_t rows, uint32_t colsSrc, uint32_t colsDst, uint8_t *q,
                            duq_stream_t stream);

/* Replaces asym_quant_host (include/quant.h:50-58, src/kernels/quant.cu:134-147):
 * unsigned nibble clamp(rint(x/scale[r]) + rint(zeros[r]), 0, 15). */
int duq_asym_quant_host(const duq_half *x, const duq_half *scale, const duq_half *zeros, uint32_t rows,
                        uint32_t colsSrc, uint32_t colsDst, uint8_t *q, duq_stream_t stream);

/* Replaces asym_dual_quant_host.  Argument order follows the DEFINITION
 * (src/kernels/quant2.cu:141-151: scale_1, zeros_1, scale_2, zeros_2) and its only caller
 * (src/export/bindings.cpp:417-420), not the differing declaration in
 * include/quant.h:92-102.  The zero is added in binary16 before rounding
 * (quant2.cu:133). */
int duq_asym_dual_quant_host(const duq_half *x, const duq_half *scale_1, const duq_half *zeros_1,
                             const duq_half *scale_2, const duq_half *zeros_2, uint32_t rows,
                             uint32_t colsSrc, uint32_t colsDst, uint8_t *q, duq_stream_t stream);

/* ---- fused per-token quantizers (scale computed in the same pass) -------------------- */

/* One pass over x replacing SymQuantizer.forward (qlinear4bit/nn/quantizer.py:10-16;
 * C++ Quantizer4bit::forward, src/module/quant_tensor.cu:151-161), i.e. the ~5 torch ops
 * for the scale plus sym_quant_host:
 *   scale[r] = h(h(max_k|x[r,k]| / 7) * clip),  q as duq_sym_quant_host_qmax.
 * x rows must be 16-byte aligned (cols % 8 == 0 and x 16-byte aligned); cols even. */
int duq_quantize_rows_sym(const duq_half *x, uint32_t rows, uint32_t cols, float clip, int32_t qmax,
                          uint8_t *q, duq_half *scale, duq_stream_t stream);

/* One pass replacing AsymQuantizer.forward (qlinear4bit/nn/quantizer.py:24-35):
 *   scale[r] = h(h(max-min)/15), zeros[r] = h(rint(h(h(-min)/scale[r]))), q as
 * duq_asym_quant_host.  Same alignment rules as duq_quantize_rows_sym. */
int duq_quantize_rows_asym(const duq_half *x, uint32_t rows, uint32_t cols, uint8_t *q, duq_half *scale,
                           duq_half *zeros, duq_stream_t stream);

/* Signed-shifted form of duq_quantize_rows_asym for the row-sum epilogue (no counterpart in
 * the reference, whose unsigned codes are misread by its signed GEMM, README.md:31-32):
 * same scale and the same codes u as duq_quantize_rows_asym, stored as the signed nibble
 * u - 8; zeros[r] = h(zero - 8); rowsum[r] = sum_k (u[r,k] - 8).  Then
 * x[r,k] ~ scale[r] * (s4(q[r,k]) - zeros[r]) and the signed GEMM is exact for it. */
int duq_quantize_rows_asym_shifted(const duq_half *x, uint32_t rows, uint32_t cols, uint8_t *q,
                                   duq_half *scale, duq_half *zeros, int32_t *rowsum, duq_stream_t stream);

/* ---- GEMM ---------------------------------------------------------------------------- */

/* Replaces matmul_host_4bit (include/gemm.h:5-12, src/kernels/gemm.cu:8-43):
 * C[m,n] = sum_k s4(A[m,k]) * s4(B[n,k]), A [M,K/2] and B [N,K/2] row-major packed,
 * C [M,N] row-major int32, both operands read as SIGNED nibbles.  K % 64 == 0
 * (qlinear4bit/tools/tensor_utils.py:52); A, B rows 16-byte aligned follows from that
 * when A and B are 16-byte aligned, which is required.  Exact for K <= 131008. */
int duq_matmul_host_4bit(const uint8_t *A, const uint8_t *B, uint32_t M, uint32_t N, uint32_t K,
                         int32_t *C, duq_stream_t stream);

/* Replaces batch_matmul_host_4bit (include/gemm.h:23-31, src/kernels/gemm.cu:83-117; binding batched_matmul,
 * src/export/bindings.cpp:46-86): batch_count problems of one shape in ONE launch,
 * C[i] = s4(A[i]) * s4(B[i])^T.  The reference takes arrays of per-problem pointers that its only caller fills
 * with base + i * stride of contiguous tensors (bindings.cpp:67-71); here the three tensors are passed as such:
 * A [batch_count, M, K/2], B [batch_count, N, K/2], C [batch_count, M, N], contiguous.  Same K rules as
 * duq_matmul_host_4bit (K % 64 == 0 keeps every problem 16-byte aligned). */
int duq_batch_matmul_host_4bit(const uint8_t *A, const uint8_t *B, uint32_t M, uint32_t N, uint32_t K,
                               int32_t *C, uint32_t batch_count, duq_stream_t stream);

/* ---- stand-alone dequant epilogues (int32 accumulators in HBM -> fp16) ---------------- */

/* Replaces sym_dequant_host (include/quant.h:19-26, src/kernels/quant.cu:83-97):
 * x[r,c] = h(h(scale_row[r]*scale_col[c]) * h_rn(q[r,c])). */
int duq_sym_dequant_host(const int32_t *q, const duq_half *scale_row, const duq_half *scale_col,
                         uint32_t rows, uint32_t cols, duq_half *x, duq_stream_t stream);

/* Replaces sym_dual_dequant_host (include/quant.h:40-48, src/kernels/quant2.cu:85-98):
 * column scale = c < 10 ? scale_col_1[c] : scale_col_2[c]. */
int duq_sym_dual_dequant_host(const int32_t *q, const duq_half *scale_row, const duq_half *scale_col_1,
                              const duq_half *scale_col_2, uint32_t rows, uint32_t cols, duq_half *x,
                              duq_stream_t stream);

/* Replaces asym_dequant_host (include/quant.h:60-69, src/kernels/quant.cu:171-188):
 * x = h(h(s_r*s_c) * h(h(h_rn(q) - z_r) - z_c)). */
int duq_asym_dequant_host(const int32_t *q, const duq_half *scale_row, const duq_half *zeros_row,
                          const duq_half *scale_col, const duq_half *zeros_col, uint32_t rows,
                          uint32_t cols, duq_half *x, duq_stream_t stream);

/* Replaces asym_dual_dequant_host (include/quant.h:105-116, src/kernels/quant2.cu:188-208):
 * the column selector of the reference kernel is non-zero for column 0 only
 * (quant2.cu:182-183), so column 0 uses (scale_col_1, zeros_col_1) and every other
 * column (scale_col_2, zeros_col_2). */
int duq_asym_dual_dequant_host(const int32_t *q, const duq_half *scale_row, const duq_half *zeros_row,
                               const duq_half *scale_col_1, const duq_half *zeros_col_1,
                               const duq_half *scale_col_2, const duq_half *zeros_col_2, uint32_t rows,
                               uint32_t cols, duq_half *x, duq_stream_t stream);

/* Replaces asym_batch_dequant_host (include/quant.h:80-90, src/kernels/quant.cu:190-239): the asymmetric
 * epilogue of duq_asym_dequant_host over q [batches, rows, cols] in one launch, batch entry b reading
 * scale_row / zeros_row [b * rows + r] and scale_col / zeros_col [b * cols + c]. */
int duq_asym_batch_dequant_host(const int32_t *q, const duq_half *scale_row, const duq_half *zeros_row,
                                const duq_half *scale_col, const duq_half *zeros_col, uint32_t batches,
                                uint32_t rows, uint32_t cols, duq_half *x, duq_stream_t stream);

/* ---- fused GEMM + dequant (+ bias) ---------------------------------------------------- */

/* One launch replacing matmul_host_4bit + {sym,asym,sym_dual,asym_dual}_dequant_host and
 * the trailing torch `+ bias` of the module forwards (qlinear4bit/nn/linear.py:42-56,
 * 104-115,167-176,239-250; C++ Linear4bit::forward, src/module/linear.cu:108-153):
 * the int32 accumulators never go to HBM.  Results are bit-identical to the unfused
 * sequence.
 *   mode       DUQ_EPI_*
 *   xq         [M,K/2] packed activations, scale_x [M], zeros_x [M] (asym modes, else NULL)
 *   w          [N,K/2] packed weights
 *   w_scale_1  [N]; w_zeros_1 [N] (asym modes); w_scale_2 / w_zeros_2 [N] (dual modes)
 *   bias       [N] or NULL;  y [M,N] fp16 row-major
 * K % 64 == 0; xq, w 16-byte aligned. */
int duq_linear4bit_forward(int32_t mode, const uint8_t *xq, const duq_half *scale_x, const duq_half *zeros_x,
                           const uint8_t *w, const duq_half *w_scale_1, const duq_half *w_zeros_1,
                           const duq_half *w_scale_2, const duq_half *w_zeros_2, const duq_half *bias,
                           uint32_t M, uint32_t N, uint32_t K, duq_half *y, duq_stream_t stream);

/* duq_linear4bit_forward over batch_count problems of one shape in ONE launch: what the loop of
 * AsymQuantMatMul.forward (qlinear4bit/nn/matmul.py:55-63: a GEMM per batch entry into an int32 tensor, then
 * asym_batch_dequant) and a batched SymQuantMatMul compute, without the int32 tensor.  Every tensor is
 * contiguous over the batch: xq [batch_count, M, K/2], w [batch_count, N, K/2], per-row parameters
 * [batch_count, M], per-column parameters and bias [batch_count, N], y [batch_count, M, N].  Bit-identical to
 * batch_count calls of duq_linear4bit_forward. */
int duq_batch_linear4bit_forward(int32_t mode, const uint8_t *xq, const duq_half *scale_x, const duq_half *zeros_x,
                                 const uint8_t *w, const duq_half *w_scale_1, const duq_half *w_zeros_1,
                                 const duq_half *w_scale_2, const duq_half *w_zeros_2, const duq_half *bias,
                                 uint32_t batch_count, uint32_t M, uint32_t N, uint32_t K, duq_half *y,
                                 duq_stream_t stream);

/* Which kernel family duq_matmul_host_4bit / duq_linear4bit_forward run for a shape (no GPU work; for tests
 * and tuning): 1 decode rows kernel (M <= 4), 2 decode MFMA kernel (M <= 16; up to 64 rows of at most 8192
 * elements, 48 of at most 12288), 3 dot kernel (M <= 4, rows longer than 16384 elements), 4 ring kernel, 5 skinny
 * kernel (9 <= M <= 16, very wide problems), 6 stream kernel (prefill), 7 tile kernel.  Families 1-5 address the weight tensor with 32-bit byte offsets and are only picked while
 * N * K / 2 < 2^32 - 256; larger tensors run the stream / tile kernels, whose bases are 64-bit per tile.  No
 * counterpart in the reference (CUTLASS picks its own tile, src/kernels/gemm.cu:17-42). */
int duq_gemm_kernel_for(uint32_t M, uint32_t N, uint32_t K);
/* For a shape of family 6: the stream kernel's tile as rows * 1000 + columns (256256, 128256, 64256, 32256, 128128,
 * 64128); 0 for the other families.  (The dual-uniform row-sum epilogue never runs the 256-row tile.) */
int duq_gemm_stream_tile_for(uint32_t M, uint32_t N, uint32_t K);

/* Measurement aid, no counterpart in the reference: reads `bytes` (16-byte aligned, < 4 GiB) of device memory
 * with the access pattern of the decode kernels (every load of a workgroup requested up front, 32 KB per
 * workgroup) and discards them; `sink` (64 words, may be NULL) only keeps the loads alive.  Its duration for
 * N * K / 2 bytes is the floor of a decode launch over weights of that size (bench.py reports it beside every
 * decode row). */
int duq_probe_read(const void *src, uint64_t bytes, uint32_t *sink, duq_stream_t stream);

/* ---- quantize + GEMM + dequant (+ bias) from binary16 activations ---------------------- */

/* No counterpart in the reference, where this is SymQuantizer.forward followed by Linear4bitSQ.forward /
 * Linear4bitDUSQ.forward (qlinear4bit/nn/quantizer.py:10-16, qlinear4bit/nn/linear.py:42-56, 167-176: ~5 torch
 * ops, sym_quant, matmul, sym_dequant, + bias).  y is bit-identical to duq_quantize_rows_sym followed by
 * duq_linear4bit_forward:
 *   x [M,K] binary16, 16-byte aligned;  clip, qmax as duq_quantize_rows_sym
 *   mode DUQ_EPI_SYM (w_scale_2 NULL) or DUQ_EPI_SYM_DUAL;  w, w_scale_1, w_scale_2, bias, y as duq_linear4bit_forward
 *   q_out [M,K/2] / scale_out [M]: optional (NULL): the packed codes and per-token scales, for callers that need
 *   them as well
 * Up to four rows (K <= 16384, N * K / 2 < 2^32 - 256; from two rows on K <= 8192 or N <= 16384), five to eight rows
 * of at most 4096 elements (8192 with N <= 4096) and nine to sixteen rows that hold at most 32768 elements together (40960
 * with N <= 4096; K <= 4096, N <= 16384) run as ONE launch: every workgroup quantizes the rows itself while its
 * weights are in flight, and `workspace` is not touched.  Any other shape runs two launches
 * (quantizer, then GEMM) and stages the codes and scales in `workspace`, device memory of at least
 * duq_quantize_linear4bit_workspace_bytes(M, N, K) bytes (0 for the one-launch shapes), 16-byte aligned, that the
 * caller provides and may reuse once the call's work has completed on the stream (DUQ_E_NULL / DUQ_E_SHAPE if it
 * is missing or too small; codes and scales go to q_out / scale_out instead when both are given). */
uint64_t duq_quantize_linear4bit_workspace_bytes(uint32_t M, uint32_t N, uint32_t K);
int duq_quantize_linear4bit_forward(int32_t mode, const duq_half *x, float clip, int32_t qmax, const uint8_t *w,
                                    const duq_half *w_scale_1, const duq_half *w_scale_2, const duq_half *bias,
                                    uint32_t M, uint32_t N, uint32_t K, duq_half *y, uint8_t *q_out,
                                    duq_half *scale_out, void *workspace, uint64_t workspace_bytes,
                                    duq_stream_t stream);

/* The same from binary16 activations for the asymmetric layers (no counterpart in the reference, where this is
 * AsymQuantizer.forward followed by Linear4bitASQ.forward / LinearQuant4bitDUASQ.forward,
 * qlinear4bit/nn/quantizer.py:24-35, qlinear4bit/nn/linear.py:104-115, 239-250), and for the row-sum mode:
 *   mode DUQ_EPI_ASYM       y = duq_quantize_rows_asym, then duq_linear4bit_forward(DUQ_EPI_ASYM), bit for bit
 *        DUQ_EPI_ASYM_DUAL  the same with the dual-uniform epilogue (w_scale_2, w_zeros_2)
 *        DUQ_EPI_ASYM_ROWSUM  duq_quantize_rows_asym_shifted, then duq_linear4bit_forward_rowsum (w_rowsum_adj)
 *        DUQ_EPI_ASYM_DUAL_ROWSUM  duq_quantize_rows_asym_shifted, then duq_linear4bit_forward_dual_rowsum
 *                           (w_rowsum_adj = its w_adj_1, w_rowsum_adj_2 = its w_adj_2)
 *   q_out [M,K/2], scale_out [M], zeros_out [M], rowsum_out [M] (row-sum modes): optional (NULL)
 * The shapes that run as ONE launch are those of duq_quantize_linear4bit_forward; the others run quantizer + GEMM
 * and stage codes, scales, zero points (and row sums; in the dual-uniform row-sum mode also the int32 accumulators,
 * for shapes whose GEMM cannot apply that epilogue itself) in `workspace`
 * (duq_quantize_linear4bit_asym_workspace_bytes(mode, M, N, K) bytes, 16-byte aligned; whatever the caller's own
 * output pointers cover is written there instead). */
uint64_t duq_quantize_linear4bit_asym_workspace_bytes(int32_t mode, uint32_t M, uint32_t N, uint32_t K);
int duq_quantize_linear4bit_forward_asym(int32_t mode, const duq_half *x, const uint8_t *w, const duq_half *w_scale_1,
                                         const duq_half *w_zeros_1, const duq_half *w_scale_2,
                                         const duq_half *w_zeros_2, const int32_t *w_rowsum_adj,
                                         const int32_t *w_rowsum_adj_2, const duq_half *bias, uint32_t M, uint32_t N,
                                         uint32_t K, duq_half *y, uint8_t *q_out, duq_half *scale_out,
                                         duq_half *zeros_out, int32_t *rowsum_out, void *workspace,
                                         uint64_t workspace_bytes, duq_stream_t stream);

/* The two entry points above with the layer's side of the arguments in a struct the caller fills once per layer
 * (no counterpart in the reference): a decode step then passes seven arguments instead of seventeen to twenty, which
 * is what a step costs on the host when it goes through a foreign-function interface (ctypes: about 0.1 us per
 * argument).  Shapes that run as ONE launch take no workspace (NULL, 0); the others stage what the quantizer
 * launch hands to the GEMM launch in `workspace`, of duq_quantize_linear4bit_workspace_bytes(M, N, K) bytes for the
 * symmetric modes and duq_quantize_linear4bit_asym_workspace_bytes(mode, M, N, K) for the others, 16-byte aligned
 * (DUQ_E_NULL without one, DUQ_E_SHAPE for one that is too small, before anything is launched).
 *   mode  DUQ_EPI_SYM / DUQ_EPI_SYM_DUAL (clip, qmax as duq_quantize_rows_sym) or one of the asymmetric modes of
 *         duq_quantize_linear4bit_forward_asym (clip, qmax ignored); pointers a mode does not use are NULL */
typedef struct duq_fused_layer {
    int32_t mode;
    float clip;
    int32_t qmax;
    uint32_t N, K;
    const uint8_t *w;
    const duq_half *w_scale_1, *w_zeros_1, *w_scale_2, *w_zeros_2;
    const int32_t *w_rowsum_adj, *w_rowsum_adj_2;
    const duq_half *bias;
} duq_fused_layer;
int duq_quantize_linear4bit_forward_layer(const duq_fused_layer *layer, const duq_half *x, uint32_t M, duq_half *y,
                                          void *workspace, uint64_t workspace_bytes, duq_stream_t stream);

/* No counterpart in the reference.  For callers that cannot allocate device memory or carry a workspace around
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc):
 * duq_quantize_linear4bit_forward without the workspace arguments.  The codes and scales that its quantizer
 * launch hands to its GEMM launch are staged in a device array that is part of the library's code object:
 * DUQ_STATIC_SCRATCH_SLOTS slots of DUQ_STATIC_SCRATCH_CODE_BYTES + 2 * DUQ_STATIC_SCRATCH_ROWS bytes (33 MiB in
 * all; every GPU the library runs on holds its own copy until the process ends).  The call allocates and frees
 * nothing.  y (and q_out / scale_out) are bit-identical to duq_quantize_linear4bit_forward's.
 *   limit   M * K / 2 <= DUQ_STATIC_SCRATCH_CODE_BYTES and M <= DUQ_STATIC_SCRATCH_ROWS, whatever the launch plan,
 *           else DUQ_E_SCRATCH (e.g. 4096 x 4096 or 2048 x 8192 activations fit, 4096 x 8192 do not)
 *   slot    which slot the call stages in, 0 .. DUQ_STATIC_SCRATCH_SLOTS - 1 (else DUQ_E_SCRATCH).  Calls whose work
 *           may overlap in time on one GPU (different streams, graphs replayed concurrently) must use different
 *           slots: two overlapping calls on one slot race on it with no error.  Calls ordered on one stream may
 *           share a slot.  Nothing in a slot has to start at zero: each call overwrites the part it reads.
 *   device  the stream must belong to the current device (DUQ_E_DEVICE otherwise).  The first staged call on a
 *           device asks the runtime for the array's address (hipGetSymbolAddress), which a stream under capture
 *           may not do: such a call returns DUQ_E_CAPTURE.  duq_static_scratch_init() does the lookup for the
 *           current device up front; afterwards a call reads one atomic pointer and takes no lock. */
#define DUQ_STATIC_SCRATCH_CODE_BYTES (8u << 20)
#define DUQ_STATIC_SCRATCH_ROWS 32768u
#define DUQ_STATIC_SCRATCH_SLOTS 4u
int duq_static_scratch_init(void);
int duq_quantize_linear4bit_forward_static(int32_t mode, const duq_half *x, float clip, int32_t qmax, const uint8_t *w,
                                           const duq_half *w_scale_1, const duq_half *w_scale_2, const duq_half *bias,
                                           uint32_t M, uint32_t N, uint32_t K, duq_half *y, uint8_t *q_out,
                                           duq_half *scale_out, uint32_t slot, duq_stream_t stream);

/* ---- asymmetric forward with exact zero-point correction (row sums) -------------------- */

/* No counterpart in the reference (its asymmetric epilogue, src/kernels/quant.cu:167-168,
 * subtracts the zero points from the accumulator, which is not the correction).  Operands
 * hold signed-shifted codes c with shifted zero points z, x[m,k] ~ s_x[m]*(c_x[m,k] - z_x[m])
 * and w[n,k] ~ s_w[n]*(c_w[n,k] - z_w[n]), so that
 *   sum_k x*w = s_x*s_w * (acc - z_x*(R_w[n] - K*z_w[n]) - z_w[n]*R_x[m]),  R = sum_k c.
 *   rowsum_x      [M] int32  R_x, as written by duq_quantize_rows_asym_shifted
 *   w_rowsum_adj  [N] int32  R_w[n] - K*z_w[n], computed once with the weights
 * The correction is evaluated in wrapping 32-bit integers (zero points are integer-valued
 * binary16 numbers, converted with round-to-nearest), then
 *   y = h(f32(f32(corr) * (f32(s_x)*f32(s_w))));  with bias: y = h(y + bias[n]).
 * Same shape and alignment rules as duq_linear4bit_forward. */
int duq_linear4bit_forward_rowsum(const uint8_t *xq, const duq_half *scale_x, const duq_half *zeros_x,
                                  const int32_t *rowsum_x, const uint8_t *w, const duq_half *w_scale,
                                  const duq_half *w_zeros, const int32_t *w_rowsum_adj, const duq_half *bias,
                                  uint32_t M, uint32_t N, uint32_t K, duq_half *y, duq_stream_t stream);

/* The same epilogue on int32 accumulators already in HBM (q [rows, cols] from
 * duq_matmul_host_4bit); bit-identical to duq_linear4bit_forward_rowsum. */
int duq_asym_rowsum_dequant_host(const int32_t *q, const duq_half *scale_row, const duq_half *zeros_row,
                                 const int32_t *rowsum_row, const duq_half *scale_col, const duq_half *zeros_col,
                                 const int32_t *rowsum_adj_col, const duq_half *bias, uint32_t rows, uint32_t cols,
                                 duq_half *x, duq_stream_t stream);

/* Row-sum epilogue for the dual-uniform layer (no counterpart in the reference).  LinearQuant4bitDUASQ
 * (qlinear4bit/nn/linear.py:252-297) quantizes input columns 0..9 of every weight row with (scale_1, zero_1) and
 * the others with (scale_2, zero_2); the reference epilogue (src/kernels/quant2.cu:158-186) applies ONE of the two
 * pairs per output column (its selector is non-zero for output column 0 only) to the whole accumulator, which is
 * not the product of the dequantized operands.  That product needs the accumulator split at input column 10:
 *   accL = sum_{k<10} c_x[m,k] c_w[n,k],  accR = q[m,n] - accL,  R_xL = sum_{k<10} c_x[m,k],  R_xR = rowsum_row[m] - R_xL
 *   corrL = accL - z_x[m]*adj_col_1[n] - z_1[n]*R_xL      adj_col_1[n] = sum_{k<10}  c_w[n,k] - 10*z_1[n]
 *   corrR = accR - z_x[m]*adj_col_2[n] - z_2[n]*R_xR      adj_col_2[n] = sum_{k>=10} c_w[n,k] - (K-10)*z_2[n]
 *   x[m,n] = h( f32(corrL)*(f32(s_x)*f32(s_1)) + f32(corrR)*(f32(s_x)*f32(s_2)) )   (+ bias: h(x + bias[n]))
 * with every float32 operator rounded, corrections in wrapping 32-bit integers, codes and zero points signed-shifted
 * as for duq_linear4bit_forward_rowsum (activations from duq_quantize_rows_asym_shifted).
 *   q    [rows, cols] int32 from duq_matmul_host_4bit(xq, w)
 *   xq   [rows, K/2], w [cols, K/2]: the packed operands of that GEMM; the first eight bytes of every row are read
 *        (16-byte aligned, K % 64 == 0) */
int duq_asym_dual_rowsum_dequant_host(const int32_t *q, const uint8_t *xq, const duq_half *scale_row,
                                      const duq_half *zeros_row, const int32_t *rowsum_row, const uint8_t *w,
                                      const duq_half *scale_col_1, const duq_half *zeros_col_1,
                                      const duq_half *scale_col_2, const duq_half *zeros_col_2,
                                      const int32_t *adj_col_1, const int32_t *adj_col_2, const duq_half *bias,
                                      uint32_t rows, uint32_t cols, uint32_t K, duq_half *x, duq_stream_t stream);

/* GEMM + that epilogue: y[M,N] = dual row-sum epilogue of xq[M,K/2] x w[N,K/2]^T, bit-identical to
 * duq_matmul_host_4bit followed by duq_asym_dual_rowsum_dequant_host (no counterpart in the reference).  Shapes for
 * which duq_linear4bit_dual_rowsum_workspace_bytes(M, N, K) is 0 (the decode kernels, up to 64 rows, and the prefill
 * kernel with rows longer than 256 elements and N % 8 == 0) run as one launch and `acc_workspace` may be NULL; the others run those two launches and
 * stage the int32 accumulators in `acc_workspace` (at least the bytes the query returns, 16-byte aligned, owned by
 * the caller: the library allocates nothing).  y 16-byte aligned, the column arrays as torch allocates them
 * (16-byte aligned). */
uint64_t duq_linear4bit_dual_rowsum_workspace_bytes(uint32_t M, uint32_t N, uint32_t K);
int duq_linear4bit_forward_dual_rowsum(const uint8_t *xq, const duq_half *scale_x, const duq_half *zeros_x,
                                       const int32_t *rowsum_x, const uint8_t *w, const duq_half *w_scale_1,
                                       const duq_half *w_zeros_1, const duq_half *w_scale_2,
                                       const duq_half *w_zeros_2, const int32_t *w_adj_1, const int32_t *w_adj_2,
                                       const duq_half *bias, uint32_t M, uint32_t N, uint32_t K, duq_half *y,
                                       void *acc_workspace, uint64_t workspace_bytes, duq_stream_t stream);

/* ---- the same forward on the 6-bit float matrix path ---------------------------------- */

/* No counterpart in the reference.  Every int4 value is exactly an E3M2 ("bf6") number and
 * the float32 accumulation of their products is exact below 2^24 (|C| <= 64*K), so the
 * MFMA for 6-bit floats, which runs at twice the rate of the 8-bit integer one, returns the
 * integer GEMM bit for bit.  The operands are shadows of the packed-int4 tensors, 3/4 byte per
 * element, in a layout private to the library:
 *   duq_weight_shadow_bf6      w    [N,K/2] -> w_bf6 [ceil(N/32)*32*K*3/4 bytes], once per weight tensor
 *   duq_activation_shadow_bf6  xq   [M,K/2] -> x_bf6 [M*K*3/4 bytes] (the *_bf6 quantizers
 *                              below write it directly)
 * duq_linear4bit_forward_bf6 takes the shadows in place of xq and w, and otherwise the
 * arguments of duq_linear4bit_forward (modes DUQ_EPI_SYM .. DUQ_EPI_ASYM_DUAL) or of
 * duq_linear4bit_forward_rowsum (mode DUQ_EPI_ASYM_ROWSUM: rowsum_x, w_rowsum_adj; NULL in
 * the other modes); y is bit-identical to theirs.
 * K % 128 == 0, N % 16 == 0; shadows and y 16-byte aligned, per-column arrays 8-byte
 * aligned (w_rowsum_adj 16). */
int duq_weight_shadow_bf6(const uint8_t *w, uint32_t N, uint32_t K, uint8_t *w_bf6, duq_stream_t stream);
/* duq_quantize_rows_sym / duq_quantize_rows_asym (rowsum NULL) / duq_quantize_rows_asym_shifted
 * (rowsum given) that also write the shadow of the codes; q may be NULL when only the shadow is
 * wanted.  cols % 128 == 0. */
int duq_quantize_rows_sym_bf6(const duq_half *x, uint32_t rows, uint32_t cols, float clip, int32_t qmax, uint8_t *q,
                              uint8_t *x_bf6, duq_half *scale, duq_stream_t stream);
int duq_quantize_rows_asym_bf6(const duq_half *x, uint32_t rows, uint32_t cols, uint8_t *q, uint8_t *x_bf6,
                               duq_half *scale, duq_half *zeros, int32_t *rowsum, duq_stream_t stream);
int duq_activation_shadow_bf6(const uint8_t *xq, uint32_t M, uint32_t K, uint8_t *x_bf6, duq_stream_t stream);
int duq_linear4bit_forward_bf6(int32_t mode, const uint8_t *x_bf6, const duq_half *scale_x, const duq_half *zeros_x,
                               const int32_t *rowsum_x, const uint8_t *w_bf6, const duq_half *w_scale_1,
                               const duq_half *w_zeros_1, const duq_half *w_scale_2, const duq_half *w_zeros_2,
                               const int32_t *w_rowsum_adj, const duq_half *bias, uint32_t M, uint32_t N, uint32_t K,
                               duq_half *y, duq_stream_t stream);

/* duq_linear4bit_forward_dual_rowsum on the 6-bit float matrix path (no counterpart in the reference): the GEMM reads
 * the shadows, the epilogue (inside the same launch) the first eight bytes of every row of the packed operands the
 * shadows were made from, xq [M,K/2] and w [N,K/2] (the codes of input columns 0..9).  y is bit-identical to
 * duq_linear4bit_forward_dual_rowsum's.  K % 128 == 0, N % 16 == 0; shadows, packed operands and y 16-byte aligned. */
int duq_linear4bit_forward_dual_rowsum_bf6(const uint8_t *x_bf6, const uint8_t *xq, const duq_half *scale_x,
                                           const duq_half *zeros_x, const int32_t *rowsum_x, const uint8_t *w_bf6,
                                           const uint8_t *w, const duq_half *w_scale_1, const duq_half *w_zeros_1,
                                           const duq_half *w_scale_2, const duq_half *w_zeros_2, const int32_t *w_adj_1,
                                           const int32_t *w_adj_2, const duq_half *bias, uint32_t M, uint32_t N,
                                           uint32_t K, duq_half *y, duq_stream_t stream);

/* ---- the 8-bit asymmetric layer (LinearQuant8bitASQ, qlinear4bit/nn/linear.py:300-368) ---- */

/* float32 activations [rows, cols], per-row float32 scale and zero point ->
 * int8 codes clamp(rint(half(x / scale)) + rint(half(zero)), 0, 126).
 * Replaces asym_quant_host_8bit (include/quant.h:71, src/kernels/quant.cu:241-279;
 * binding src/export/bindings.cpp:245-266). */
int duq_asym_quant_host_8bit(const float *x, const float *scale, const float *zeros, uint32_t rows, uint32_t cols,
                             int8_t *q, duq_stream_t stream);

/* A [M,K] int8 times B [N,K] int8 (both row-major; B is the weight as stored) -> C [M,N]
 * int32, K % 32 == 0, K <= 131040 (no accumulator can overflow, so the result does not depend on whether the
 * matrix unit wraps or saturates), A and B 16-byte aligned.
 * Replaces matmul_host_8bit (include/gemm.h:14, src/kernels/gemm.cu:46-81; binding
 * src/export/bindings.cpp:28-45; the Python wrapper asserts K % 32 == 0,
 * qlinear4bit/tools/tensor_utils.py:57-61). */
int duq_matmul_host_8bit(const int8_t *A, const int8_t *B, uint32_t M, uint32_t N, uint32_t K, int32_t *C,
                         duq_stream_t stream);

/* x[r,c] = (scale_row[r] * scale_col[c]) * (float(q[r,c]) - (zeros_row[r] + zeros_col[c])), float32
 * with one rounding per operator.
 * Replaces asym_dequant_host_hprec (include/quant.h:118, src/kernels/quant.cu:281-323;
 * binding src/export/bindings.cpp:309-350). */
int duq_asym_dequant_host_hprec(const int32_t *q, const float *scale_row, const float *zeros_row,
                                const float *scale_col, const float *zeros_col, uint32_t rows, uint32_t cols, float *x,
                                duq_stream_t stream);

/* No counterpart in the reference: AsymQuantizer8bit.forward (qlinear4bit/nn/quantizer.py:38-55)
 * in one launch: per-row min / max, scale = (max - min) / 127, zero = rint(-min / scale), then
 * the codes of duq_asym_quant_host_8bit.  cols % 4 == 0, x 16-byte aligned, q 4-byte aligned. */
int duq_quantize_rows_asym_8bit(const float *x, uint32_t rows, uint32_t cols, int8_t *q, float *scale, float *zeros,
                                duq_stream_t stream);

/* No counterpart in the reference: duq_matmul_host_8bit + duq_asym_dequant_host_hprec (+ float32
 * bias [N], may be NULL) in one launch, the accumulators never leaving the registers;
 * y [M,N] float32 is bit-identical to the three steps (LinearQuant8bitASQ.forward,
 * qlinear4bit/nn/linear.py:323-335). */
int duq_linear8bit_forward(const int8_t *xq, const float *scale_x, const float *zeros_x, const int8_t *w,
                           const float *w_scale, const float *w_zeros, const float *bias, uint32_t M, uint32_t N,
                           uint32_t K, float *y, duq_stream_t stream);

/* No counterpart in the reference: the same forward on a weight copy arranged for the MFMA operand layout.
 * duq_weight_tile_8bit rewrites w [N,K] once into w_tiled, ceil(N/32)*32*K bytes (whole 32-row tiles, the
 * last one zero-padded), in which the 64 x 16 bytes a wavefront loads for one MFMA are one contiguous
 * kilobyte; duq_linear8bit_forward_tiled takes it in place of w and returns the same bits, faster (the
 * row-major form touches four times as many cache lines per load).  K % 32 == 0; 16-byte alignment. */
int duq_weight_tile_8bit(const int8_t *w, uint32_t N, uint32_t K, int8_t *w_tiled, duq_stream_t stream);
int duq_linear8bit_forward_tiled(const int8_t *xq, const float *scale_x, const float *zeros_x, const int8_t *w_tiled,
                                 const float *w_scale, const float *w_zeros, const float *bias, uint32_t M, uint32_t N,
                                 uint32_t K, float *y, duq_stream_t stream);

/* No counterpart in the reference: LinearQuant8bitASQ.forward with its own quantizer (qlinear4bit/nn/linear.py:323-335)
 * in one call: duq_quantize_rows_asym_8bit into `workspace`, then duq_linear8bit_forward(_tiled) on it; the same
 * bits as the two calls.  x [M,K] float32, 16-byte aligned, K % 32 == 0; w the weight as stored and / or w_tiled its
 * tiled copy (one may be NULL): up to four rows (two of more than 4096 elements) read w when it is given, everything
 * else w_tiled when it is given.  workspace: duq_quantize_linear8bit_workspace_bytes(M, K) bytes (codes, scales,
 * zero points), 16-byte aligned.  What a step of the layer costs at a few rows is mostly the host's share of a
 * call; this halves it. */
uint64_t duq_quantize_linear8bit_workspace_bytes(uint32_t M, uint32_t K);
int duq_quantize_linear8bit_forward(const float *x, const int8_t *w, const int8_t *w_tiled, const float *w_scale,
                                    const float *w_zeros, const float *bias, uint32_t M, uint32_t N, uint32_t K, float *y,
                                    void *workspace, uint64_t workspace_bytes, duq_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* DUQ_HIP_H */
