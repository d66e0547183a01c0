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

}  // namespace duq
