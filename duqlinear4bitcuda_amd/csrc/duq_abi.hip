// extern "C" boundary of libduq_hip.so: argument validation, then the launchers.
// Nothing here allocates, synchronises or throws; the only state is the per-device address of the static
// scratch array of duq_quantize_linear4bit_forward_static.
#include <atomic>

#include "../../include/duq_hip.h"
#include "duq_launch.h"

// Scratch of duq_quantize_linear4bit_forward_static: DUQ_STATIC_SCRATCH_SLOTS slots, each the packed codes
// [M, K/2] and then the per-token scales [M] that the call's quantizer launch hands to its GEMM launch.  Every GPU
// the library runs on holds its own copy of the array until the process ends.  In host code the name is only a
// handle for hipGetSymbolAddress: kernels and copies get the device address that static_scratch() looks up once per
// device.
constexpr uint64_t kSlotBytes = (uint64_t)DUQ_STATIC_SCRATCH_CODE_BYTES + DUQ_STATIC_SCRATCH_ROWS * 2;
static __device__ __align__(256) unsigned char scratch[DUQ_STATIC_SCRATCH_SLOTS * kSlotBytes];

namespace {

constexpr int kMaxDevices = 64;
std::atomic<void *> g_scratch_ptr[kMaxDevices];  // device address of `scratch` on device i, null until first use there

// Address of `scratch` on the device of `stream`, which must be the current device (the lookup and the launches
// that follow act on the current device).  The first call per device asks the runtime, which a stream under
// capture may not do: such a call is refused instead (call duq_static_scratch_init first).  Later calls read one
// atomic pointer.  Two threads that race on the first call both look the address up and store the same value.
int static_scratch(hipStream_t stream, unsigned char **out)
{
    int dev = -1;
    if (hipError_t e = hipGetDevice(&dev)) return static_cast<int>(e);
    if (dev < 0 || dev >= kMaxDevices) return static_cast<int>(hipErrorInvalidDevice);
    if (stream) {
        hipDevice_t sdev = -1;
        if (hipError_t e = hipStreamGetDevice(stream, &sdev)) return static_cast<int>(e);
        if (static_cast<int>(sdev) != dev) return DUQ_E_DEVICE;
    }
    void *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        if (stream) {
            hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
            if (hipError_t e = hipStreamIsCapturing(stream, &cap)) return static_cast<int>(e);
            if (cap != hipStreamCaptureStatusNone) return DUQ_E_CAPTURE;
        }
        if (hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch))) return static_cast<int>(e);
        if (!p) return static_cast<int>(hipErrorInvalidSymbol);
        g_scratch_ptr[dev].store(p, std::memory_order_release);
    }
    *out = static_cast<unsigned char *>(p);
    return DUQ_OK;
}

inline hipStream_t as_stream(duq_stream_t s) { return reinterpret_cast<hipStream_t>(s); }
inline bool aligned(const void *p, uintptr_t a) { return reinterpret_cast<uintptr_t>(p) % a == 0; }

int check_quant_shape(uint32_t rows, uint32_t colsSrc, uint32_t colsDst)
{
    (void)rows;
    if (colsDst != (colsSrc + 1) / 2) return DUQ_E_SHAPE;
    return DUQ_OK;
}

int check_qmax(int32_t qmax) { return (qmax >= 0 && qmax <= 7) ? DUQ_OK : DUQ_E_MODE; }

int check_gemm(const void *A, const void *B, uint32_t M, uint32_t N, uint32_t K)
{
    if (M == 0 || N == 0) return DUQ_OK;
    if (!A || !B) return DUQ_E_NULL;
    if (K % 64 != 0) return DUQ_E_KALIGN;
    // K: accumulators are carried x256 in int32 (or as float32 integers below 2^24); M, N: the kernels index one
    // output tile's rows with 32-bit byte offsets (256 rows x N x 4 bytes)
    if (K > 131008u || N > (1u << 22) || M > (1u << 24)) return DUQ_E_TOO_LARGE;
    if (!aligned(A, 16) || !aligned(B, 16)) return DUQ_E_ALIGN;
    return DUQ_OK;
}

// quantize + GEMM + dequant from binary16 activations: one launch for decode shapes, otherwise the quantizer
// into `workspace` (codes, scales, then zero points and row sums for the asymmetric modes) followed by the GEMM.
// The epilogue mode decides the quantizer: symmetric for DUQ_EPI_SYM / SYM_DUAL, asymmetric for DUQ_EPI_ASYM /
// ASYM_DUAL, its signed-shifted form for DUQ_EPI_ASYM_ROWSUM.
struct FusedOut {
    uint8_t *q;
    duq_half *scale, *zeros;
    int32_t *rowsum;
};

inline uint64_t up16(uint64_t v) { return (v + 15) & ~(uint64_t)15; }

// codes, scales, zero points (asymmetric modes), row sums (row-sum modes), and for the dual-uniform row-sum mode
// on a shape whose GEMM cannot apply that epilogue itself the int32 accumulators
uint64_t staging_bytes(int32_t mode, uint32_t M, uint32_t N, uint32_t K)
{
    uint64_t b = up16((uint64_t)M * (K / 2)) + up16((uint64_t)M * 2);
    if (mode == DUQ_EPI_ASYM || mode == DUQ_EPI_ASYM_DUAL || mode >= DUQ_EPI_ASYM_ROWSUM) b += up16((uint64_t)M * 2);
    if (mode >= DUQ_EPI_ASYM_ROWSUM) b += up16((uint64_t)M * 4);
    if (mode == DUQ_EPI_ASYM_DUAL_ROWSUM && !duq::gemm_fuses_dual_rowsum(M, N, K)) b += up16((uint64_t)M * N * 4);
    return b;
}

int quantize_linear_impl(duq::Epilogue e, const duq_half *x, float clip, int32_t qmax, const uint8_t *w, uint32_t M,
                         uint32_t N, uint32_t K, duq_half *y, FusedOut out, void *workspace, uint64_t workspace_bytes,
                         duq_stream_t stream)
{
    const int32_t mode = e.mode;
    const bool asym = mode == DUQ_EPI_ASYM || mode == DUQ_EPI_ASYM_DUAL || mode >= DUQ_EPI_ASYM_ROWSUM;
    const bool dual = mode == DUQ_EPI_SYM_DUAL || mode == DUQ_EPI_ASYM_DUAL || mode == DUQ_EPI_ASYM_DUAL_ROWSUM;
    const bool rowsum = mode >= DUQ_EPI_ASYM_ROWSUM;
    if (mode < DUQ_EPI_SYM || mode > DUQ_EPI_ASYM_DUAL_ROWSUM) return DUQ_E_MODE;
    if (int st = check_qmax(qmax)) return st;
    if (M == 0 || N == 0) return DUQ_OK;
    if (!x) return DUQ_E_NULL;
    if (int st = check_gemm(x, w, M, N, K)) return st;
    if (K == 0) return DUQ_E_KALIGN;
    if (!e.s_col_1 || !y) return DUQ_E_NULL;
    if (asym && !e.z_col_1) return DUQ_E_NULL;
    if (dual && (!e.s_col_2 || (asym && !e.z_col_2))) return DUQ_E_NULL;
    if (rowsum && !e.rs_col) return DUQ_E_NULL;
    if (mode == DUQ_EPI_ASYM_DUAL_ROWSUM && !e.rs_col_2) return DUQ_E_NULL;
    if ((out.q && !aligned(out.q, 16))) return DUQ_E_ALIGN;
    if (duq::decode_fp16in_one_launch(M, N, K))
        return duq::launch_decode_fp16in(x, clip, qmax, w, M, N, K, e, y, out.q, out.scale, asym ? out.zeros : nullptr,
                                         rowsum ? out.rowsum : nullptr, as_stream(stream));
    // two launches: codes and per-token parameters go to the caller's outputs where given, else to the workspace
    const bool acc_ws = mode == DUQ_EPI_ASYM_DUAL_ROWSUM && !duq::gemm_fuses_dual_rowsum(M, N, K);
    const bool need_ws = !out.q || !out.scale || (asym && !out.zeros) || (rowsum && !out.rowsum) || acc_ws;
    int32_t *acc = nullptr;
    if (need_ws) {
        if (!workspace) return DUQ_E_NULL;
        if (!aligned(workspace, 16)) return DUQ_E_ALIGN;
        if (workspace_bytes < staging_bytes(mode, M, N, K)) return DUQ_E_SHAPE;
        uint8_t *at = static_cast<uint8_t *>(workspace);
        if (!out.q) out.q = at;
        at += up16((uint64_t)M * (K / 2));
        if (!out.scale) out.scale = reinterpret_cast<duq_half *>(at);
        at += up16((uint64_t)M * 2);
        if (asym && !out.zeros) out.zeros = reinterpret_cast<duq_half *>(at);
        at += up16((uint64_t)M * 2);
        if (rowsum && !out.rowsum) out.rowsum = reinterpret_cast<int32_t *>(at);
        at += up16((uint64_t)M * 4);
        if (acc_ws) acc = reinterpret_cast<int32_t *>(at);
    }
    int st;
    if (!asym)
        st = duq::launch_quantize_rows_sym(x, M, K, clip, qmax, out.q, out.scale, nullptr, as_stream(stream));
    else
        st = duq::launch_quantize_rows_asym(x, M, K, out.q, out.scale, out.zeros, rowsum ? out.rowsum : nullptr, nullptr,
                                            as_stream(stream));
    if (st) return st;
    e.s_row = out.scale;
    e.z_row = asym ? out.zeros : nullptr;
    e.rs_row = rowsum ? out.rowsum : nullptr;
    if (acc_ws) {  // GEMM into int32, then the stand-alone epilogue
        if (int st2 = duq::launch_gemm_s4(out.q, w, M, N, K, acc, nullptr, nullptr, as_stream(stream))) return st2;
        duq::DualRowsumParams dp{acc,       out.q,     w,         K / 2,    out.scale, out.zeros, out.rowsum, e.s_col_1, e.z_col_1,
                                 e.s_col_2, e.z_col_2, e.rs_col,  e.rs_col_2, e.bias,  M,         N,          y};
        return duq::launch_dual_rowsum_dequant(dp, as_stream(stream));
    }
    return duq::launch_gemm_s4(out.q, w, M, N, K, nullptr, &e, y, as_stream(stream));
}

}  // namespace

extern "C" {

int duq_abi_version(void) { return 1; }

const char *duq_status_string(int status)
{
    switch (status) {
    case DUQ_OK: return "ok";
    case DUQ_E_NULL: return "a required pointer is NULL";
    case DUQ_E_SHAPE: return "inconsistent dimensions";
    case DUQ_E_KALIGN: return "K must be a multiple of 64 (packed row length a multiple of 32 bytes); 128 on the 6-bit float path, 32 on the 8-bit one";
    case DUQ_E_MODE: return "unknown epilogue mode or unsupported qmax";
    case DUQ_E_ALIGN: return "pointer alignment requirement not met";
    case DUQ_E_TOO_LARGE: return "dimension too large";
    case DUQ_E_SCRATCH:
        return "input exceeds a slot of the static scratch buffer (M * K / 2 <= 8 MiB of packed codes and M <= 32768 rows), or no such slot";
    case DUQ_E_DEVICE: return "the stream belongs to another device than the current one";
    case DUQ_E_CAPTURE:
        return "first use of the static scratch buffer on this device under stream capture: call duq_static_scratch_init() before capturing";
    default: break;
    }
    if (status > 0) return hipGetErrorString(static_cast<hipError_t>(status));
    return "unknown status";
}

int duq_get_dual_quant_col_k(void) { return DUQ_QUANT_COL_K; }

int duq_sym_quant_host_qmax(const duq_half *x, const duq_half *scale, uint32_t rows, uint32_t colsSrc,
                            uint32_t colsDst, int32_t qmax, uint8_t *q, duq_stream_t stream)
{
    if (int e = check_quant_shape(rows, colsSrc, colsDst)) return e;
    if (int e = check_qmax(qmax)) return e;
    if (rows == 0 || colsSrc == 0) return DUQ_OK;
    if (!x || !scale || !q) return DUQ_E_NULL;
    return duq::launch_sym_quant(x, scale, rows, colsSrc, colsDst, qmax, q, as_stream(stream));
}

int duq_sym_quant_host(const duq_half *x, const duq_half *scale, uint32_t rows, uint32_t colsSrc, uint32_t colsDst,
                       uint8_t *q, duq_stream_t stream)
{
    return duq_sym_quant_host_qmax(x, scale, rows, colsSrc, colsDst, DUQ_QMAX_SYM_DEVICE, q, stream);
}

int duq_sym_dual_quant_host(const duq_half *x, const duq_half *scale_1, const duq_half *scale_2, uint32_t rows,
                            uint32_t colsSrc, uint32_t colsDst, uint8_t *q, duq_stream_t stream)
{
    if (int e = check_quant_shape(rows, colsSrc, colsDst)) return e;
    if (rows == 0 || colsSrc == 0) return DUQ_OK;
    if (!x || !scale_1 || !scale_2 || !q) return DUQ_E_NULL;
    return duq::launch_sym_dual_quant(x, scale_1, scale_2, rows, colsSrc, colsDst, DUQ_QMAX_SYM_DEVICE, q,
                                      as_stream(stream));
}

int duq_asym_quant_host(const duq_half *x, const duq_half *scale, const duq_half *zeros, uint32_t rows,
                        uint32_t colsSrc, uint32_t colsDst, uint8_t *q, duq_stream_t stream)
{
    if (int e = check_quant_shape(rows, colsSrc, colsDst)) return e;
    if (rows == 0 || colsSrc == 0) return DUQ_OK;
    if (!x || !scale || !zeros || !q) return DUQ_E_NULL;
    return duq::launch_asym_quant(x, scale, zeros, rows, colsSrc, colsDst, q, as_stream(stream));
}

int duq_asym_dual_quant_host(const duq_half *x, const duq_half *scale_1, const duq_half *zeros_1,
                             const duq_half *scale_2, const duq_half *zeros_2, uint32_t rows, uint32_t colsSrc,
                             uint32_t colsDst, uint8_t *q, duq_stream_t stream)
{
    if (int e = check_quant_shape(rows, colsSrc, colsDst)) return e;
    if (rows == 0 || colsSrc == 0) return DUQ_OK;
    if (!x || !scale_1 || !zeros_1 || !scale_2 || !zeros_2 || !q) return DUQ_E_NULL;
    return duq::launch_asym_dual_quant(x, scale_1, zeros_1, scale_2, zeros_2, rows, colsSrc, colsDst, q,
                                       as_stream(stream));
}

int duq_quantize_rows_sym(const duq_half *x, uint32_t rows, uint32_t cols, float clip, int32_t qmax, uint8_t *q,
                          duq_half *scale, duq_stream_t stream)
{
    if (int e = check_qmax(qmax)) return e;
    if (rows == 0 || cols == 0) return DUQ_OK;
    if (!x || !q || !scale) return DUQ_E_NULL;
    if (cols % 32 != 0) return DUQ_E_SHAPE;
    if (!aligned(x, 16) || !aligned(q, 16)) return DUQ_E_ALIGN;
    return duq::launch_quantize_rows_sym(x, rows, cols, clip, qmax, q, scale, nullptr, as_stream(stream));
}

int duq_quantize_rows_asym(const duq_half *x, uint32_t rows, uint32_t cols, uint8_t *q, duq_half *scale,
                           duq_half *zeros, duq_stream_t stream)
{
    if (rows == 0 || cols == 0) return DUQ_OK;
    if (!x || !q || !scale || !zeros) return DUQ_E_NULL;
    if (cols % 32 != 0) return DUQ_E_SHAPE;
    if (!aligned(x, 16) || !aligned(q, 16)) return DUQ_E_ALIGN;
    return duq::launch_quantize_rows_asym(x, rows, cols, q, scale, zeros, nullptr, nullptr, as_stream(stream));
}

int duq_quantize_rows_asym_shifted(const duq_half *x, uint32_t rows, uint32_t cols, uint8_t *q, duq_half *scale,
                                   duq_half *zeros, int32_t *rowsum, duq_stream_t stream)
{
    if (rows == 0 || cols == 0) return DUQ_OK;
    if (!x || !q || !scale || !zeros || !rowsum) return DUQ_E_NULL;
    if (cols % 32 != 0) return DUQ_E_SHAPE;
    if (!aligned(x, 16) || !aligned(q, 16)) return DUQ_E_ALIGN;
    return duq::launch_quantize_rows_asym(x, rows, cols, q, scale, zeros, rowsum, nullptr, as_stream(stream));
}

int duq_matmul_host_4bit(const uint8_t *A, const uint8_t *B, uint32_t M, uint32_t N, uint32_t K, int32_t *C,
                         duq_stream_t stream)
{
    if (int e = check_gemm(A, B, M, N, K)) return e;
    if (M == 0 || N == 0) return DUQ_OK;
    if (!C) return DUQ_E_NULL;
    return duq::launch_gemm_s4(A, B, M, N, K, C, nullptr, nullptr, as_stream(stream));
}

int duq_sym_dequant_host(const int32_t *q, const duq_half *scale_row, const duq_half *scale_col, uint32_t rows,
                         uint32_t cols, duq_half *x, duq_stream_t stream)
{
    if (rows == 0 || cols == 0) return DUQ_OK;
    if (!q || !scale_row || !scale_col || !x) return DUQ_E_NULL;
    duq::Epilogue e{DUQ_EPI_SYM, scale_row, nullptr, scale_col, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
    return duq::launch_dequant(q, e, rows, cols, x, as_stream(stream));
}

int duq_sym_dual_dequant_host(const int32_t *q, const duq_half *scale_row, const duq_half *scale_col_1,
                              const duq_half *scale_col_2, uint32_t rows, uint32_t cols, duq_half *x,
                              duq_stream_t stream)
{
    if (rows == 0 || cols == 0) return DUQ_OK;
    if (!q || !scale_row || !scale_col_1 || !scale_col_2 || !x) return DUQ_E_NULL;
    duq::Epilogue e{DUQ_EPI_SYM_DUAL, scale_row, nullptr, scale_col_1, nullptr, scale_col_2, nullptr, nullptr, nullptr, nullptr};
    return duq::launch_dequant(q, e, rows, cols, x, as_stream(stream));
}

int duq_asym_dequant_host(const int32_t *q, const duq_half *scale_row, const duq_half *zeros_row,
                          const duq_half *scale_col, const duq_half *zeros_col, uint32_t rows, uint32_t cols,
                          duq_half *x, duq_stream_t stream)
{
    if (rows == 0 || cols == 0) return DUQ_OK;
    if (!q || !scale_row || !zeros_row || !scale_col || !zeros_col || !x) return DUQ_E_NULL;
    duq::Epilogue e{DUQ_EPI_ASYM, scale_row, zeros_row, scale_col, zeros_col, nullptr, nullptr, nullptr, nullptr, nullptr};
    return duq::launch_dequant(q, e, rows, cols, x, as_stream(stream));
}

int duq_asym_dual_dequant_host(const int32_t *q, const duq_half *scale_row, const duq_half *zeros_row,
                               const duq_half *scale_col_1, const duq_half *zeros_col_1, const duq_half *scale_col_2,
                               const duq_half *zeros_col_2, uint32_t rows, uint32_t cols, duq_half *x,
                               duq_stream_t stream)
{
    if (rows == 0 || cols == 0) return DUQ_OK;
    if (!q || !scale_row || !zeros_row || !scale_col_1 || !zeros_col_1 || !scale_col_2 || !zeros_col_2 || !x)
        return DUQ_E_NULL;
    duq::Epilogue e{DUQ_EPI_ASYM_DUAL, scale_row, zeros_row, scale_col_1, zeros_col_1, scale_col_2, zeros_col_2,
                    nullptr, nullptr, nullptr};
    return duq::launch_dequant(q, e, rows, cols, x, as_stream(stream));
}

int duq_linear4bit_forward(int32_t mode, const uint8_t *xq, const duq_half *scale_x, const duq_half *zeros_x,
                           const uint8_t *w, const duq_half *w_scale_1, const duq_half *w_zeros_1,
                           const duq_half *w_scale_2, const duq_half *w_zeros_2, const duq_half *bias, uint32_t M,
                           uint32_t N, uint32_t K, duq_half *y, duq_stream_t stream)
{
    if (mode < DUQ_EPI_SYM || mode > DUQ_EPI_ASYM_DUAL) return DUQ_E_MODE;
    if (int e = check_gemm(xq, w, M, N, K)) return e;
    if (M == 0 || N == 0) return DUQ_OK;
    if (!scale_x || !w_scale_1 || !y) return DUQ_E_NULL;
    const bool asym = mode == DUQ_EPI_ASYM || mode == DUQ_EPI_ASYM_DUAL;
    const bool dual = mode == DUQ_EPI_SYM_DUAL || mode == DUQ_EPI_ASYM_DUAL;
    if (asym && (!zeros_x || !w_zeros_1)) return DUQ_E_NULL;
    if (dual && !w_scale_2) return DUQ_E_NULL;
    if (asym && dual && !w_zeros_2) return DUQ_E_NULL;
    duq::Epilogue e{mode, scale_x, zeros_x, w_scale_1, w_zeros_1, w_scale_2, w_zeros_2, bias, nullptr, nullptr};
    return duq::launch_gemm_s4(xq, w, M, N, K, nullptr, &e, y, as_stream(stream));
}

// One launch holds at most 65535 batch entries (grid limit of the second and third dimension): longer batches
// run in slices, every tensor moved on by whole entries.
constexpr uint32_t kBatchSlice = 65535;

static void advance(duq::Epilogue &e, uint64_t entries, uint32_t rows, uint32_t cols)
{
    const uint64_t r = entries * rows, c = entries * cols;
    if (e.s_row) e.s_row += r;
    if (e.z_row) e.z_row += r;
    if (e.rs_row) e.rs_row += r;
    if (e.s_col_1) e.s_col_1 += c;
    if (e.z_col_1) e.z_col_1 += c;
    if (e.s_col_2) e.s_col_2 += c;
    if (e.z_col_2) e.z_col_2 += c;
    if (e.bias) e.bias += c;
    if (e.rs_col) e.rs_col += c;
}

int duq_batch_matmul_host_4bit(const uint8_t *A, const uint8_t *B, uint32_t M, uint32_t N, uint32_t K, int32_t *C,
                               uint32_t batch_count, duq_stream_t stream)
{
    if (batch_count == 0) return DUQ_OK;
    if (int e = check_gemm(A, B, M, N, K)) return e;
    if (M == 0 || N == 0) return DUQ_OK;
    if (!C) return DUQ_E_NULL;
    for (uint32_t b0 = 0; b0 < batch_count; b0 += kBatchSlice) {
        const uint32_t nb = batch_count - b0 < kBatchSlice ? batch_count - b0 : kBatchSlice;
        if (int st = duq::launch_gemm_s4_batched(A + (uint64_t)b0 * M * (K / 2), B + (uint64_t)b0 * N * (K / 2), M, N, K,
                                                 nb, C + (uint64_t)b0 * M * N, nullptr, nullptr, as_stream(stream)))
            return st;
    }
    return DUQ_OK;
}

int duq_asym_batch_dequant_host(const int32_t *q, const duq_half *scale_row, const duq_half *zeros_row,
                                const duq_half *scale_col, const duq_half *zeros_col, uint32_t batches,
                                uint32_t rows, uint32_t cols, duq_half *x, duq_stream_t stream)
{
    if (batches == 0 || rows == 0 || cols == 0) return DUQ_OK;
    if (!q || !scale_row || !zeros_row || !scale_col || !zeros_col || !x) return DUQ_E_NULL;
    duq::Epilogue e{DUQ_EPI_ASYM, scale_row, zeros_row, scale_col, zeros_col, nullptr, nullptr, nullptr, nullptr, nullptr};
    for (uint32_t b0 = 0; b0 < batches; b0 += kBatchSlice) {
        const uint32_t nb = batches - b0 < kBatchSlice ? batches - b0 : kBatchSlice;
        if (int st = duq::launch_dequant_batched(q + (uint64_t)b0 * rows * cols, e, nb, rows, cols,
                                                 x + (uint64_t)b0 * rows * cols, as_stream(stream)))
            return st;
        advance(e, nb, rows, cols);
    }
    return DUQ_OK;
}

int duq_batch_linear4bit_forward(int32_t mode, const uint8_t *xq, const duq_half *scale_x, const duq_half *zeros_x,
                                 const uint8_t *w, const duq_half *w_scale_1, const duq_half *w_zeros_1,
                                 const duq_half *w_scale_2, const duq_half *w_zeros_2, const duq_half *bias,
                                 uint32_t batch_count, uint32_t M, uint32_t N, uint32_t K, duq_half *y,
                                 duq_stream_t stream)
{
    if (mode < DUQ_EPI_SYM || mode > DUQ_EPI_ASYM_DUAL) return DUQ_E_MODE;
    if (batch_count == 0) return DUQ_OK;
    if (int e = check_gemm(xq, w, M, N, K)) return e;
    if (M == 0 || N == 0) return DUQ_OK;
    if (!scale_x || !w_scale_1 || !y) return DUQ_E_NULL;
    const bool asym = mode == DUQ_EPI_ASYM || mode == DUQ_EPI_ASYM_DUAL;
    const bool dual = mode == DUQ_EPI_SYM_DUAL || mode == DUQ_EPI_ASYM_DUAL;
    if (asym && (!zeros_x || !w_zeros_1)) return DUQ_E_NULL;
    if (dual && !w_scale_2) return DUQ_E_NULL;
    if (asym && dual && !w_zeros_2) return DUQ_E_NULL;
    duq::Epilogue e{mode, scale_x, zeros_x, w_scale_1, w_zeros_1, w_scale_2, w_zeros_2, bias, nullptr, nullptr};
    for (uint32_t b0 = 0; b0 < batch_count; b0 += kBatchSlice) {
        const uint32_t nb = batch_count - b0 < kBatchSlice ? batch_count - b0 : kBatchSlice;
        if (int st = duq::launch_gemm_s4_batched(xq + (uint64_t)b0 * M * (K / 2), w + (uint64_t)b0 * N * (K / 2), M, N, K,
                                                 nb, nullptr, &e, y + (uint64_t)b0 * M * N, as_stream(stream)))
            return st;
        advance(e, nb, M, N);
    }
    return DUQ_OK;
}

int duq_probe_read(const void *src, uint64_t bytes, uint32_t *sink, duq_stream_t stream)
{
    if (bytes == 0) return DUQ_OK;
    if (!src) return DUQ_E_NULL;
    if (!aligned(src, 16)) return DUQ_E_ALIGN;
    if (bytes >= 0xFFFFFF00ull) return DUQ_E_TOO_LARGE;
    return duq::launch_probe_read(src, bytes, sink, as_stream(stream));
}

int duq_gemm_kernel_for(uint32_t M, uint32_t N, uint32_t K) { return duq::select_gemm_kernel(M, N, K); }

int duq_gemm_stream_tile_for(uint32_t M, uint32_t N, uint32_t K)
{
    if (duq::select_gemm_kernel(M, N, K) != duq::kKernelStream) return 0;
    const duq::StreamTile t = duq::select_stream_tile(M, N, K, 1, false);
    return (int)(t.rows * 1000 + t.cols);
}

uint64_t duq_quantize_linear4bit_workspace_bytes(uint32_t M, uint32_t N, uint32_t K)
{
    if (M == 0 || N == 0 || K == 0) return 0;
    if (duq::decode_fp16in_one_launch(M, N, K)) return 0;  // nothing staged
    // packed codes [M, K/2] (rounded up to 16 bytes so that the scales stay aligned), then the scales [M]
    return staging_bytes(DUQ_EPI_SYM, M, N, K);
}

int duq_quantize_linear4bit_forward(int32_t mode, const duq_half *x, float clip, int32_t qmax, const uint8_t *w,
                                    const duq_half *w_scale_1, const duq_half *w_scale_2, const duq_half *bias,
                                    uint32_t M, uint32_t N, uint32_t K, duq_half *y, uint8_t *q_out,
                                    duq_half *scale_out, void *workspace, uint64_t workspace_bytes,
                                    duq_stream_t stream)
{
    if (mode != DUQ_EPI_SYM && mode != DUQ_EPI_SYM_DUAL) return DUQ_E_MODE;
    duq::Epilogue e{mode, nullptr, nullptr, w_scale_1, nullptr, w_scale_2, nullptr, bias, nullptr, nullptr};
    return quantize_linear_impl(e, x, clip, qmax, w, M, N, K, y, FusedOut{q_out, scale_out, nullptr, nullptr}, workspace,
                                workspace_bytes, stream);
}

uint64_t duq_quantize_linear4bit_asym_workspace_bytes(int32_t mode, uint32_t M, uint32_t N, uint32_t K)
{
    if (M == 0 || N == 0 || K == 0) return 0;
    if (mode != DUQ_EPI_ASYM && mode != DUQ_EPI_ASYM_DUAL && mode != DUQ_EPI_ASYM_ROWSUM && mode != DUQ_EPI_ASYM_DUAL_ROWSUM)
        return 0;
    if (duq::decode_fp16in_one_launch(M, N, K)) return 0;
    return staging_bytes(mode, M, N, K);
}

int duq_quantize_linear4bit_forward_asym(int32_t mode, const duq_half *x, const uint8_t *w, const duq_half *w_scale_1,
                                         const duq_half *w_zeros_1, const duq_half *w_scale_2,
                                         const duq_half *w_zeros_2, const int32_t *w_rowsum_adj,
                                         const int32_t *w_rowsum_adj_2, const duq_half *bias, uint32_t M, uint32_t N,
                                         uint32_t K, duq_half *y, uint8_t *q_out, duq_half *scale_out,
                                         duq_half *zeros_out, int32_t *rowsum_out, void *workspace,
                                         uint64_t workspace_bytes, duq_stream_t stream)
{
    if (mode != DUQ_EPI_ASYM && mode != DUQ_EPI_ASYM_DUAL && mode != DUQ_EPI_ASYM_ROWSUM && mode != DUQ_EPI_ASYM_DUAL_ROWSUM)
        return DUQ_E_MODE;
    duq::Epilogue e{mode,      nullptr, nullptr, w_scale_1,    w_zeros_1,     w_scale_2,
                    w_zeros_2, bias,    nullptr, w_rowsum_adj, w_rowsum_adj_2};
    return quantize_linear_impl(e, x, 1.0f, DUQ_QMAX_SYM_DEVICE, w, M, N, K, y, FusedOut{q_out, scale_out, zeros_out, rowsum_out},
                                workspace, workspace_bytes, stream);
}

int duq_quantize_linear4bit_forward_layer(const duq_fused_layer *layer, const duq_half *x, uint32_t M, duq_half *y,
                                          void *workspace, uint64_t workspace_bytes, duq_stream_t stream)
{
    if (!layer) return DUQ_E_NULL;
    const duq_fused_layer &l = *layer;
    if (l.mode < DUQ_EPI_SYM || l.mode > DUQ_EPI_ASYM_DUAL_ROWSUM) return DUQ_E_MODE;
    if (M == 0 || l.N == 0) return DUQ_OK;
    if (l.K == 0) return DUQ_E_SHAPE;
    const bool sym = l.mode == DUQ_EPI_SYM || l.mode == DUQ_EPI_SYM_DUAL;
    duq::Epilogue e{l.mode,      nullptr, nullptr, l.w_scale_1,    sym ? nullptr : l.w_zeros_1, l.w_scale_2,
                    sym ? nullptr : l.w_zeros_2, l.bias,  nullptr, l.w_rowsum_adj, l.w_rowsum_adj_2};
    return quantize_linear_impl(e, x, sym ? l.clip : 1.0f, sym ? l.qmax : DUQ_QMAX_SYM_DEVICE, l.w, M, l.N, l.K, y,
                                FusedOut{nullptr, nullptr, nullptr, nullptr}, workspace, workspace_bytes, stream);
}

int duq_static_scratch_init(void)
{
    unsigned char *p = nullptr;
    return static_scratch(nullptr, &p);
}

int duq_quantize_linear4bit_forward_static(int32_t mode, const duq_half *x, float clip, int32_t qmax, const uint8_t *w,
                                           const duq_half *w_scale_1, const duq_half *w_scale_2, const duq_half *bias,
                                           uint32_t M, uint32_t N, uint32_t K, duq_half *y, uint8_t *q_out,
                                           duq_half *scale_out, uint32_t slot, duq_stream_t stream)
{
    // Same work as duq_quantize_linear4bit_forward with the staging buffer taken from `scratch`.  The size is
    // checked first, for every shape, so that what a caller may pass does not depend on the launch plan.
    if (mode != DUQ_EPI_SYM && mode != DUQ_EPI_SYM_DUAL) return DUQ_E_MODE;
    if (slot >= DUQ_STATIC_SCRATCH_SLOTS) return DUQ_E_SCRATCH;
    if ((uint64_t)M * (K / 2) > DUQ_STATIC_SCRATCH_CODE_BYTES || M > DUQ_STATIC_SCRATCH_ROWS) return DUQ_E_SCRATCH;
    uint8_t *q = q_out;
    duq_half *sc = scale_out;
    const bool staged = M != 0 && N != 0 && K != 0 && !duq::decode_fp16in_one_launch(M, N, K) && (!q_out || !scale_out);
    if (staged) {
        unsigned char *ws = nullptr;
        if (int e = static_scratch(as_stream(stream), &ws)) return e;
        ws += (uint64_t)slot * kSlotBytes;
        // codes at the start of the slot, scales behind the largest code block: both offsets keep the 256-byte alignment
        if (!q) q = ws;
        if (!sc) sc = reinterpret_cast<duq_half *>(ws + DUQ_STATIC_SCRATCH_CODE_BYTES);
    }
    duq::Epilogue e{mode, nullptr, nullptr, w_scale_1, nullptr, w_scale_2, nullptr, bias, nullptr, nullptr};
    return quantize_linear_impl(e, x, clip, qmax, w, M, N, K, y, FusedOut{q, sc, nullptr, nullptr}, nullptr, 0, stream);
}

int duq_asym_rowsum_dequant_host(const int32_t *q, const duq_half *scale_row, const duq_half *zeros_row,
                                 const int32_t *rowsum_row, const duq_half *scale_col, const duq_half *zeros_col,
                                 const int32_t *rowsum_adj_col, const duq_half *bias, uint32_t rows, uint32_t cols,
                                 duq_half *x, duq_stream_t stream)
{
    if (rows == 0 || cols == 0) return DUQ_OK;
    if (!q || !scale_row || !zeros_row || !rowsum_row || !scale_col || !zeros_col || !rowsum_adj_col || !x)
        return DUQ_E_NULL;
    duq::Epilogue e{DUQ_EPI_ASYM_ROWSUM, scale_row, zeros_row, scale_col, zeros_col, nullptr, nullptr, bias,
                    rowsum_row, rowsum_adj_col};
    return duq::launch_dequant(q, e, rows, cols, x, as_stream(stream));
}

int duq_asym_dual_rowsum_dequant_host(const int32_t *q, const uint8_t *xq, const duq_half *scale_row,
                                      const duq_half *zeros_row, const int32_t *rowsum_row, const uint8_t *w,
                                      const duq_half *scale_col_1, const duq_half *zeros_col_1,
                                      const duq_half *scale_col_2, const duq_half *zeros_col_2,
                                      const int32_t *adj_col_1, const int32_t *adj_col_2, const duq_half *bias,
                                      uint32_t rows, uint32_t cols, uint32_t K, duq_half *x, duq_stream_t stream)
{
    if (int e = check_gemm(xq, w, rows, cols, K)) return e;
    if (rows == 0 || cols == 0) return DUQ_OK;
    if (K == 0) return DUQ_E_KALIGN;
    if (!q || !scale_row || !zeros_row || !rowsum_row || !scale_col_1 || !zeros_col_1 || !scale_col_2 || !zeros_col_2 ||
        !adj_col_1 || !adj_col_2 || !x)
        return DUQ_E_NULL;
    duq::DualRowsumParams p{q,           xq,          w,           K / 2,     scale_row, zeros_row, rowsum_row, scale_col_1,
                            zeros_col_1, scale_col_2, zeros_col_2, adj_col_1, adj_col_2, bias,      rows,       cols,
                            x};
    return duq::launch_dual_rowsum_dequant(p, as_stream(stream));
}

uint64_t duq_linear4bit_dual_rowsum_workspace_bytes(uint32_t M, uint32_t N, uint32_t K)
{
    if (M == 0 || N == 0 || K == 0) return 0;
    return duq::gemm_fuses_dual_rowsum(M, N, K) ? 0 : (uint64_t)M * N * 4;
}

int duq_linear4bit_forward_dual_rowsum(const uint8_t *xq, const duq_half *scale_x, const duq_half *zeros_x,
                                       const int32_t *rowsum_x, const uint8_t *w, const duq_half *w_scale_1,
                                       const duq_half *w_zeros_1, const duq_half *w_scale_2,
                                       const duq_half *w_zeros_2, const int32_t *w_adj_1, const int32_t *w_adj_2,
                                       const duq_half *bias, uint32_t M, uint32_t N, uint32_t K, duq_half *y,
                                       void *acc_workspace, uint64_t workspace_bytes, duq_stream_t stream)
{
    if (int e = check_gemm(xq, w, M, N, K)) return e;
    if (M == 0 || N == 0) return DUQ_OK;
    if (K == 0) return DUQ_E_KALIGN;
    if (!scale_x || !zeros_x || !rowsum_x || !w_scale_1 || !w_zeros_1 || !w_scale_2 || !w_zeros_2 || !w_adj_1 || !w_adj_2 || !y)
        return DUQ_E_NULL;
    if (!aligned(y, 16)) return DUQ_E_ALIGN;
    const uint64_t need = duq_linear4bit_dual_rowsum_workspace_bytes(M, N, K);
    if (need == 0) {
        duq::Epilogue e{DUQ_EPI_ASYM_DUAL_ROWSUM, scale_x, zeros_x, w_scale_1, w_zeros_1, w_scale_2, w_zeros_2, bias, rowsum_x,
                        w_adj_1,                  w_adj_2};
        return duq::launch_gemm_s4(xq, w, M, N, K, nullptr, &e, y, as_stream(stream));
    }
    if (!acc_workspace) return DUQ_E_NULL;
    if (workspace_bytes < need) return DUQ_E_SHAPE;
    if (!aligned(acc_workspace, 16)) return DUQ_E_ALIGN;
    int32_t *acc = static_cast<int32_t *>(acc_workspace);
    if (int e = duq::launch_gemm_s4(xq, w, M, N, K, acc, nullptr, nullptr, as_stream(stream))) return e;
    duq::DualRowsumParams p{acc,       xq,        w,         K / 2,   scale_x, zeros_x, rowsum_x, w_scale_1, w_zeros_1,
                            w_scale_2, w_zeros_2, w_adj_1,   w_adj_2, bias,    M,       N,        y};
    return duq::launch_dual_rowsum_dequant(p, as_stream(stream));
}

int duq_linear4bit_forward_rowsum(const uint8_t *xq, const duq_half *scale_x, const duq_half *zeros_x,
                                  const int32_t *rowsum_x, const uint8_t *w, const duq_half *w_scale,
                                  const duq_half *w_zeros, const int32_t *w_rowsum_adj, const duq_half *bias,
                                  uint32_t M, uint32_t N, uint32_t K, duq_half *y, duq_stream_t stream)
{
    if (int e = check_gemm(xq, w, M, N, K)) return e;
    if (M == 0 || N == 0) return DUQ_OK;
    if (!scale_x || !zeros_x || !rowsum_x || !w_scale || !w_zeros || !w_rowsum_adj || !y) return DUQ_E_NULL;
    duq::Epilogue e{DUQ_EPI_ASYM_ROWSUM, scale_x, zeros_x, w_scale, w_zeros, nullptr, nullptr, bias, rowsum_x,
                    w_rowsum_adj};
    return duq::launch_gemm_s4(xq, w, M, N, K, nullptr, &e, y, as_stream(stream));
}

int duq_quantize_rows_sym_bf6(const duq_half *x, uint32_t rows, uint32_t cols, float clip, int32_t qmax, uint8_t *q,
                              uint8_t *x_bf6, duq_half *scale, duq_stream_t stream)
{
    if (int e = check_qmax(qmax)) return e;
    if (rows == 0 || cols == 0) return DUQ_OK;
    if (!x || !x_bf6 || !scale) return DUQ_E_NULL;
    if (cols % 128 != 0) return DUQ_E_SHAPE;
    if (!aligned(x, 16) || !aligned(q, 16) || !aligned(x_bf6, 16)) return DUQ_E_ALIGN;
    return duq::launch_quantize_rows_sym(x, rows, cols, clip, qmax, q, scale, x_bf6, as_stream(stream));
}

int duq_quantize_rows_asym_bf6(const duq_half *x, uint32_t rows, uint32_t cols, uint8_t *q, uint8_t *x_bf6,
                               duq_half *scale, duq_half *zeros, int32_t *rowsum, duq_stream_t stream)
{
    if (rows == 0 || cols == 0) return DUQ_OK;
    if (!x || !x_bf6 || !scale || !zeros) return DUQ_E_NULL;
    if (cols % 128 != 0) return DUQ_E_SHAPE;
    if (!aligned(x, 16) || !aligned(q, 16) || !aligned(x_bf6, 16)) return DUQ_E_ALIGN;
    return duq::launch_quantize_rows_asym(x, rows, cols, q, scale, zeros, rowsum, x_bf6, as_stream(stream));
}

int duq_weight_shadow_bf6(const uint8_t *w, uint32_t N, uint32_t K, uint8_t *w_bf6, duq_stream_t stream)
{
    if (N == 0 || K == 0) return DUQ_OK;
    if (!w || !w_bf6) return DUQ_E_NULL;
    if (K % 128 != 0) return DUQ_E_KALIGN;
    if (N % 16 != 0) return DUQ_E_SHAPE;
    if (K > 131008u) return DUQ_E_TOO_LARGE;
    if (!aligned(w, 16) || !aligned(w_bf6, 16)) return DUQ_E_ALIGN;
    return duq::launch_weight_shadow_bf6(w, N, K, w_bf6, as_stream(stream));
}

int duq_activation_shadow_bf6(const uint8_t *xq, uint32_t M, uint32_t K, uint8_t *x_bf6, duq_stream_t stream)
{
    if (M == 0 || K == 0) return DUQ_OK;
    if (!xq || !x_bf6) return DUQ_E_NULL;
    if (K % 128 != 0) return DUQ_E_KALIGN;
    if (K > 131008u) return DUQ_E_TOO_LARGE;
    if (!aligned(xq, 16) || !aligned(x_bf6, 16)) return DUQ_E_ALIGN;
    return duq::launch_activation_shadow_bf6(xq, M, K, x_bf6, as_stream(stream));
}

int duq_linear4bit_forward_bf6(int32_t mode, const uint8_t *x_bf6, const duq_half *scale_x, const duq_half *zeros_x,
                               const int32_t *rowsum_x, const uint8_t *w_bf6, const duq_half *w_scale_1,
                               const duq_half *w_zeros_1, const duq_half *w_scale_2, const duq_half *w_zeros_2,
                               const int32_t *w_rowsum_adj, const duq_half *bias, uint32_t M, uint32_t N, uint32_t K,
                               duq_half *y, duq_stream_t stream)
{
    if (mode < DUQ_EPI_SYM || mode > DUQ_EPI_ASYM_ROWSUM) return DUQ_E_MODE;
    if (M == 0 || N == 0) return DUQ_OK;
    if (!x_bf6 || !w_bf6 || !scale_x || !w_scale_1 || !y) return DUQ_E_NULL;
    if (K == 0 || K % 128 != 0) return DUQ_E_KALIGN;
    if (N % 16 != 0) return DUQ_E_SHAPE;
    if (K > 131008u || N > (1u << 22) || M > (1u << 24)) return DUQ_E_TOO_LARGE;
    const bool asym = mode == DUQ_EPI_ASYM || mode == DUQ_EPI_ASYM_DUAL || mode == DUQ_EPI_ASYM_ROWSUM;
    const bool dual = mode == DUQ_EPI_SYM_DUAL || mode == DUQ_EPI_ASYM_DUAL;
    if (asym && (!zeros_x || !w_zeros_1)) return DUQ_E_NULL;
    if (dual && !w_scale_2) return DUQ_E_NULL;
    if (asym && dual && !w_zeros_2) return DUQ_E_NULL;
    if (mode == DUQ_EPI_ASYM_ROWSUM && (!rowsum_x || !w_rowsum_adj)) return DUQ_E_NULL;
    // the kernel fetches column parameters four at a time and stores whole 16-byte pieces
    if (!aligned(x_bf6, 16) || !aligned(w_bf6, 16) || !aligned(y, 16) || !aligned(w_scale_1, 8) ||
        !aligned(w_zeros_1, 8) || !aligned(w_scale_2, 8) || !aligned(w_zeros_2, 8) || !aligned(bias, 8) ||
        !aligned(w_rowsum_adj, 16))
        return DUQ_E_ALIGN;
    duq::Epilogue e{mode, scale_x, zeros_x, w_scale_1, w_zeros_1, w_scale_2, w_zeros_2, bias, rowsum_x, w_rowsum_adj};
    return duq::launch_gemm_bf6(x_bf6, w_bf6, M, N, K, e, y, as_stream(stream));
}

int duq_linear4bit_forward_dual_rowsum_bf6(const uint8_t *x_bf6, const uint8_t *xq, const duq_half *scale_x,
                                           const duq_half *zeros_x, const int32_t *rowsum_x, const uint8_t *w_bf6,
                                           const uint8_t *w, const duq_half *w_scale_1, const duq_half *w_zeros_1,
                                           const duq_half *w_scale_2, const duq_half *w_zeros_2, const int32_t *w_adj_1,
                                           const int32_t *w_adj_2, const duq_half *bias, uint32_t M, uint32_t N,
                                           uint32_t K, duq_half *y, duq_stream_t stream)
{
    if (M == 0 || N == 0) return DUQ_OK;
    if (!x_bf6 || !xq || !w_bf6 || !w || !scale_x || !zeros_x || !rowsum_x || !w_scale_1 || !w_zeros_1 || !w_scale_2 ||
        !w_zeros_2 || !w_adj_1 || !w_adj_2 || !y)
        return DUQ_E_NULL;
    if (K == 0 || K % 128 != 0) return DUQ_E_KALIGN;
    if (N % 16 != 0) return DUQ_E_SHAPE;
    if (K > 131008u || N > (1u << 22) || M > (1u << 24)) return DUQ_E_TOO_LARGE;
    if (!aligned(x_bf6, 16) || !aligned(w_bf6, 16) || !aligned(y, 16) || !aligned(xq, 16) || !aligned(w, 16)) return DUQ_E_ALIGN;
    duq::Epilogue e{DUQ_EPI_ASYM_DUAL_ROWSUM, scale_x, zeros_x, w_scale_1, w_zeros_1, w_scale_2, w_zeros_2, bias, rowsum_x,
                    w_adj_1,                  w_adj_2};
    return duq::launch_gemm_bf6(x_bf6, w_bf6, M, N, K, e, y, as_stream(stream), xq, w);
}

// ---- 8-bit asymmetric layer ----------------------------------------------------------------

static int check_gemm8(const void *A, const void *B, uint32_t M, uint32_t N, uint32_t K)
{
    if (M == 0 || N == 0) return DUQ_OK;
    if (!A || !B) return DUQ_E_NULL;
    if (K == 0 || K % 32 != 0) return DUQ_E_KALIGN;
    // K: no int32 accumulator can overflow (|sum| <= 2^14 * K < 2^31), so wrapping (this GEMM) and saturating (the
    // reference's tensor-core GEMM) accumulation cannot differ; M, N: one tile's rows are indexed with 32-bit byte
    // offsets (128 rows x N x 4 bytes)
    if (K > 131040u || N > (1u << 22) || M > (1u << 24)) return DUQ_E_TOO_LARGE;
    if (!aligned(A, 16) || !aligned(B, 16)) return DUQ_E_ALIGN;
    return DUQ_OK;
}

int duq_asym_quant_host_8bit(const float *x, const float *scale, const float *zeros, uint32_t rows, uint32_t cols,
                             int8_t *q, duq_stream_t stream)
{
    if (rows == 0 || cols == 0) return DUQ_OK;
    if (!x || !scale || !zeros || !q) return DUQ_E_NULL;
    return duq::launch_asym_quant8(x, scale, zeros, rows, cols, q, as_stream(stream));
}

int duq_quantize_rows_asym_8bit(const float *x, uint32_t rows, uint32_t cols, int8_t *q, float *scale, float *zeros,
                                duq_stream_t stream)
{
    if (rows == 0 || cols == 0) return DUQ_OK;
    if (!x || !q || !scale || !zeros) return DUQ_E_NULL;
    if (cols % 4 != 0) return DUQ_E_SHAPE;
    if (!aligned(x, 16) || !aligned(q, 4)) return DUQ_E_ALIGN;
    return duq::launch_quantize_rows_asym8(x, rows, cols, q, scale, zeros, as_stream(stream));
}

int duq_matmul_host_8bit(const int8_t *A, const int8_t *B, uint32_t M, uint32_t N, uint32_t K, int32_t *C,
                         duq_stream_t stream)
{
    if (int e = check_gemm8(A, B, M, N, K)) return e;
    if (M == 0 || N == 0) return DUQ_OK;
    if (!C) return DUQ_E_NULL;
    if (!aligned(C, 4)) return DUQ_E_ALIGN;
    return duq::launch_gemm_s8(A, B, false, M, N, K, C, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, as_stream(stream));
}

int duq_asym_dequant_host_hprec(const int32_t *q, const float *scale_row, const float *zeros_row,
                                const float *scale_col, const float *zeros_col, uint32_t rows, uint32_t cols, float *x,
                                duq_stream_t stream)
{
    if (rows == 0 || cols == 0) return DUQ_OK;
    if (!q || !scale_row || !zeros_row || !scale_col || !zeros_col || !x) return DUQ_E_NULL;
    return duq::launch_dequant_hprec(q, scale_row, zeros_row, scale_col, zeros_col, nullptr, rows, cols, x,
                                     as_stream(stream));
}

int duq_linear8bit_forward(const int8_t *xq, const float *scale_x, const float *zeros_x, const int8_t *w,
                           const float *w_scale, const float *w_zeros, const float *bias, uint32_t M, uint32_t N,
                           uint32_t K, float *y, duq_stream_t stream)
{
    if (int e = check_gemm8(xq, w, M, N, K)) return e;
    if (M == 0 || N == 0) return DUQ_OK;
    if (!scale_x || !zeros_x || !w_scale || !w_zeros || !y) return DUQ_E_NULL;
    if (!aligned(y, 4)) return DUQ_E_ALIGN;
    return duq::launch_gemm_s8(xq, w, false, M, N, K, nullptr, scale_x, zeros_x, w_scale, w_zeros, bias, y, as_stream(stream));
}

int duq_weight_tile_8bit(const int8_t *w, uint32_t N, uint32_t K, int8_t *w_tiled, duq_stream_t stream)
{
    if (N == 0 || K == 0) return DUQ_OK;
    if (!w || !w_tiled) return DUQ_E_NULL;
    if (K % 32 != 0) return DUQ_E_KALIGN;
    if (K > 131040u || N > (1u << 22)) return DUQ_E_TOO_LARGE;
    if (!aligned(w, 16) || !aligned(w_tiled, 16)) return DUQ_E_ALIGN;
    return duq::launch_weight_tile8(w, N, K, w_tiled, as_stream(stream));
}

int duq_linear8bit_forward_tiled(const int8_t *xq, const float *scale_x, const float *zeros_x, const int8_t *w_tiled,
                                 const float *w_scale, const float *w_zeros, const float *bias, uint32_t M, uint32_t N,
                                 uint32_t K, float *y, duq_stream_t stream)
{
    if (int e = check_gemm8(xq, w_tiled, M, N, K)) return e;
    if (M == 0 || N == 0) return DUQ_OK;
    if (!scale_x || !zeros_x || !w_scale || !w_zeros || !y) return DUQ_E_NULL;
    if (!aligned(y, 4)) return DUQ_E_ALIGN;
    return duq::launch_gemm_s8(xq, w_tiled, true, M, N, K, nullptr, scale_x, zeros_x, w_scale, w_zeros, bias, y,
                               as_stream(stream));
}

uint64_t duq_quantize_linear8bit_workspace_bytes(uint32_t M, uint32_t K)
{
    return up16((uint64_t)M * K) + 2 * up16((uint64_t)M * 4);
}

int duq_quantize_linear8bit_forward(const float *x, const int8_t *w, const int8_t *w_tiled, const float *w_scale,
                                    const float *w_zeros, const float *bias, uint32_t M, uint32_t N, uint32_t K, float *y,
                                    void *workspace, uint64_t workspace_bytes, duq_stream_t stream)
{
    if (M == 0 || N == 0) return DUQ_OK;
    if (!x || (!w && !w_tiled) || !workspace) return DUQ_E_NULL;
    if (!aligned(x, 16) || !aligned(workspace, 16)) return DUQ_E_ALIGN;
    if (workspace_bytes < duq_quantize_linear8bit_workspace_bytes(M, K)) return DUQ_E_SHAPE;
    // few rows run the kernel that reads the weight as stored, the others the tiled copy when there is one
    const bool rows_kernel = w && M <= 4 && K <= (M <= 2 ? 8192u : 4096u);
    const bool tiled = w_tiled && !rows_kernel;
    const int8_t *weight = tiled ? w_tiled : w;
    if (!weight) return DUQ_E_NULL;
    int8_t *q = static_cast<int8_t *>(workspace);
    float *sx = reinterpret_cast<float *>(static_cast<uint8_t *>(workspace) + up16((uint64_t)M * K));
    float *zx = reinterpret_cast<float *>(reinterpret_cast<uint8_t *>(sx) + up16((uint64_t)M * 4));
    if (int e = check_gemm8(q, weight, M, N, K)) return e;
    if (!w_scale || !w_zeros || !y) return DUQ_E_NULL;
    if (!aligned(y, 4)) return DUQ_E_ALIGN;
    if (int e = duq::launch_quantize_rows_asym8(x, M, K, q, sx, zx, as_stream(stream))) return e;
    return duq::launch_gemm_s8(q, weight, tiled, M, N, K, nullptr, sx, zx, w_scale, w_zeros, bias, y, as_stream(stream));
}

}  // extern "C"
