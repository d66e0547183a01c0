// Stand-alone dequant kernels: int32 accumulators in HBM -> fp16, for callers that keep
// the reference's three-launch sequence (matmul, then *_dequant).  HBM-bound: 4 bytes in,
// 2 bytes out per element; 8 elements per lane step (two 128-bit loads, one 128-bit store).
#include "duq_epilogue.h"
#include "duq_launch.h"

namespace duq {

template <int MODE, bool BIAS, bool VEC>
__global__ __launch_bounds__(256) void dequant_kernel(const int32_t *__restrict__ acc, Epilogue epi, uint32_t rows,
                                                      uint32_t cols, uint16_t *__restrict__ y)
{
    constexpr int E = VEC ? 8 : 1;
    if (blockIdx.y) {  // batched launch: one accumulator matrix per blockIdx.y
        acc += (uint64_t)blockIdx.y * rows * cols;
        y += (uint64_t)blockIdx.y * rows * cols;
        batch_shift(epi, blockIdx.y, rows, cols);
    }
    const uint32_t perRow = cols / E;
    const uint64_t total = (uint64_t)rows * perRow;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (uint64_t)gridDim.x * blockDim.x) {
        const uint32_t row = (uint32_t)(i / perRow);
        const uint32_t col0 = (uint32_t)(i % perRow) * E;
        const RowEpi rp = load_row<MODE>(epi, row);
        if (VEC) {
            const v4i a0 = __builtin_nontemporal_load(reinterpret_cast<const v4i *>(acc + (uint64_t)row * cols + col0));
            const v4i a1 =
                __builtin_nontemporal_load(reinterpret_cast<const v4i *>(acc + (uint64_t)row * cols + col0 + 4));
            uint32_t out[4];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const ColParams c =
                    load_col<MODE, BIAS>(epi.s_col_1, epi.z_col_1, epi.s_col_2, epi.z_col_2, epi.bias, col0 + e, epi.rs_col);
                const uint32_t bits = dequant_one<MODE, BIAS>(e < 4 ? a0[e & 3] : a1[e & 3], rp, c);
                if (e & 1)
                    out[e >> 1] |= bits << 16;
                else
                    out[e >> 1] = bits;
            }
            *reinterpret_cast<v4u *>(y + (uint64_t)row * cols + col0) = v4u{out[0], out[1], out[2], out[3]};
        } else {
            const ColParams c =
                load_col<MODE, BIAS>(epi.s_col_1, epi.z_col_1, epi.s_col_2, epi.z_col_2, epi.bias, col0, epi.rs_col);
            y[(uint64_t)row * cols + col0] = dequant_one<MODE, BIAS>(acc[(uint64_t)row * cols + col0], rp, c);
        }
    }
}

template <int MODE, bool BIAS>
static void launch_mode(const int32_t *acc, const Epilogue &epi, uint32_t batches, uint32_t rows, uint32_t cols,
                        uint16_t *y, hipStream_t stream)
{
    // (a batch entry starts rows * cols elements after the previous one: with cols % 8 == 0 every entry keeps the
    // alignment of the first)
    const bool vec = (cols % 8 == 0) && (reinterpret_cast<uintptr_t>(acc) % 16 == 0) &&
                     (reinterpret_cast<uintptr_t>(y) % 16 == 0);
    const uint64_t total = (uint64_t)rows * (vec ? cols / 8 : cols);
    const uint32_t blocks = (uint32_t)std::min<uint64_t>((total + 255) / 256, 1u << 20);
    const dim3 grid(blocks, batches);
    if (vec)
        hipLaunchKernelGGL((dequant_kernel<MODE, BIAS, true>), grid, dim3(256), 0, stream, acc, epi, rows, cols, y);
    else
        hipLaunchKernelGGL((dequant_kernel<MODE, BIAS, false>), grid, dim3(256), 0, stream, acc, epi, rows, cols, y);
}

int launch_dequant(const int32_t *acc, const Epilogue &epi, uint32_t rows, uint32_t cols, uint16_t *y,
                   hipStream_t stream)
{
    return launch_dequant_batched(acc, epi, 1, rows, cols, y, stream);
}

int launch_dequant_batched(const int32_t *acc, const Epilogue &epi, uint32_t batches, uint32_t rows, uint32_t cols,
                           uint16_t *y, hipStream_t stream)
{
    if (rows == 0 || cols == 0 || batches == 0) return 0;
    const bool bias = epi.bias != nullptr;
#define DUQ_DQ(M)                                                          \
    case M:                                                                \
        if (bias)                                                          \
            launch_mode<M, true>(acc, epi, batches, rows, cols, y, stream);  \
        else                                                               \
            launch_mode<M, false>(acc, epi, batches, rows, cols, y, stream); \
        break;
    switch (epi.mode) {
        DUQ_DQ(0)
        DUQ_DQ(1)
        DUQ_DQ(2)
        DUQ_DQ(3)
        DUQ_DQ(4)
    default:
        return (int)hipErrorInvalidValue;
    }
#undef DUQ_DQ
    return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------------
// row-sum epilogue of the dual-uniform layer
// ---------------------------------------------------------------------------------
// A thread owns four consecutive output columns: it keeps the codes of their input columns 0..9 (two words per
// column, the second masked to its two nibbles by masking the activation side), their two scale / zero / row-sum
// pairs and the bias in registers and walks kDualRows rows; per row the workgroup needs eight bytes of the
// activation row and three parameters (the same addresses in every lane).
constexpr uint32_t kDualRows = 8;

template <bool BIAS>
__global__ __launch_bounds__(256) void dual_rowsum_dequant_kernel(DualRowsumParams p)
{
    const uint32_t n0 = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (n0 >= p.cols) return;  // (no barrier below)
    const bool vec = (p.cols % 4 == 0) && (reinterpret_cast<uintptr_t>(p.acc) % 16 == 0) &&
                     (reinterpret_cast<uintptr_t>(p.y) % 8 == 0);
    uint32_t wlo[4], whi[4];
    uint32_t z1[4], z2[4], a1[4], a2[4];
    float s1[4], s2[4];
    f16 bias[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t n = min(n0 + j, p.cols - 1);
        const v2u head = *reinterpret_cast<const v2u *>(p.w + (uint64_t)n * p.kbytes);
        wlo[j] = head[0];
        whi[j] = head[1];
        s1[j] = (float)bits_to_f16(p.s_col_1[n]);
        s2[j] = (float)bits_to_f16(p.s_col_2[n]);
        z1[j] = (uint32_t)rint_i32((float)bits_to_f16(p.z_col_1[n]));
        z2[j] = (uint32_t)rint_i32((float)bits_to_f16(p.z_col_2[n]));
        a1[j] = (uint32_t)p.adj_col_1[n];
        a2[j] = (uint32_t)p.adj_col_2[n];
        bias[j] = BIAS ? bits_to_f16(p.bias[n]) : (f16)0;
    }
    // every load of the kDualRows rows is requested before the first result is needed (rows past the end repeat
    // the last one and store nothing)
    const uint32_t r0 = blockIdx.y * kDualRows;
    v2u xh[kDualRows];
    uint32_t zxs[kDualRows], rss[kDualRows];
    float sxs[kDualRows];
    v4i accv[kDualRows];
#pragma unroll
    for (uint32_t i = 0; i < kDualRows; ++i) {
        const uint32_t r = min(r0 + i, p.rows - 1);
        xh[i] = *reinterpret_cast<const v2u *>(p.xq + (uint64_t)r * p.kbytes);
        zxs[i] = (uint32_t)rint_i32((float)bits_to_f16(p.z_row[r]));
        sxs[i] = (float)bits_to_f16(p.s_row[r]);
        rss[i] = (uint32_t)p.rs_row[r];
        if (vec) {
            accv[i] = *reinterpret_cast<const v4i *>(p.acc + (uint64_t)r * p.cols + n0);
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) accv[i][j] = p.acc[(uint64_t)r * p.cols + min(n0 + j, p.cols - 1)];
        }
    }
#pragma unroll
    for (uint32_t i = 0; i < kDualRows; ++i) {
        const uint32_t r = r0 + i;
        const uint32_t xlo = xh[i][0], xhi = xh[i][1] & 0xFFu;  // input columns 0..7 and 8, 9
        const uint32_t rxl = (uint32_t)__builtin_amdgcn_sdot8((int)xhi, 0x11111111, __builtin_amdgcn_sdot8((int)xlo, 0x11111111, 0, false), false);
        const uint32_t zx = zxs[i];
        const float sx = sxs[i];
        const uint32_t rxr = rss[i] - rxl;
        uint16_t out[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
            out[j] = dual_rowsum_one<false>(accv[i][j], xlo, xhi, zx, rxl, rxr, sx, wlo[j], whi[j], s1[j], s2[j], z1[j], z2[j],
                                            a1[j], a2[j], BIAS, bias[j]);
        if (r >= p.rows) continue;
        uint16_t *dst = p.y + (uint64_t)r * p.cols + n0;
        if (vec) {
            *reinterpret_cast<v2u *>(dst) = v2u{(uint32_t)out[0] | ((uint32_t)out[1] << 16), (uint32_t)out[2] | ((uint32_t)out[3] << 16)};
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (n0 + j < p.cols) dst[j] = out[j];
        }
    }
}

int launch_dual_rowsum_dequant(const DualRowsumParams &p, hipStream_t stream)
{
    if (p.rows == 0 || p.cols == 0) return 0;
    // at most 65535 row groups per launch (grid limit): longer inputs run in slices of rows
    constexpr uint32_t kSlice = 65535u * kDualRows;
    for (uint32_t r0 = 0; r0 < p.rows; r0 += kSlice) {
        DualRowsumParams q = p;
        q.rows = std::min(p.rows - r0, kSlice);
        q.acc += (uint64_t)r0 * p.cols;
        q.y += (uint64_t)r0 * p.cols;
        q.xq += (uint64_t)r0 * p.kbytes;
        q.s_row += r0;
        q.z_row += r0;
        q.rs_row += r0;
        const dim3 grid((p.cols + 1023) / 1024, (q.rows + kDualRows - 1) / kDualRows);
        if (p.bias)
            hipLaunchKernelGGL((dual_rowsum_dequant_kernel<true>), grid, dim3(256), 0, stream, q);
        else
            hipLaunchKernelGGL((dual_rowsum_dequant_kernel<false>), grid, dim3(256), 0, stream, q);
    }
    return (int)hipGetLastError();
}

}  // namespace duq
