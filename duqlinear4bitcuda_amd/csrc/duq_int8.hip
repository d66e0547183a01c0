// The 8-bit asymmetric layer of the reference (LinearQuant8bitASQ) for gfx950: per-token int8
// quantizer (float32 in), int8 x int8 -> int32 GEMM on v_mfma_i32_32x32x32_i8, float32
// dequant ("hprec") stand-alone or fused into the GEMM.
//   quantize : src/kernels/quant.cu:241-279      scale/zero : qlinear4bit/nn/quantizer.py:38-55
//   GEMM     : src/kernels/gemm.cu:46-81         dequant    : src/kernels/quant.cu:281-323
// Arithmetic is float32 with one rounding per operator, as in the reference; the quantizer's
// value goes through binary16 on its way to the integer (the reference passes a float to
// __half2int_rn).
#include "duq_device.h"
#include "duq_launch.h"
#include "duq_tiles.h"

// Cache policy of the decode-size kernels' weight loads: 2 = non-temporal (the weights are read once, in whole cache
// lines; measured 1-6 % faster: 16 x 11008 x 4096 10.3 against 10.85 us, 16 x 4096 x 8192 9.5 against 10.1)
#ifndef DUQ_S8_ROWS_WLOAD_AUX
#define DUQ_S8_ROWS_WLOAD_AUX 2
#endif
#ifndef DUQ_S8_DEC_WLOAD_AUX
#define DUQ_S8_DEC_WLOAD_AUX 2
#endif
#ifndef DUQ_S8_SKINNY_WLOAD_AUX
#define DUQ_S8_SKINNY_WLOAD_AUX 2
#endif

namespace duq {

typedef float v4f32 __attribute__((ext_vector_type(4)));
typedef int v16i32 __attribute__((ext_vector_type(16)));

constexpr int kQmaxAsym8 = 126;  // src/kernels/quant.cu:242

// clamp(rint(h(x / s)) + zi, 0, 126); the add wraps like the 32-bit add of the reference
__device__ __forceinline__ uint32_t asym8_code(float x, float s, int zi)
{
    const f16 hq = (f16)(x / s);  // IEEE float32 quotient, then one rounding to binary16
    const int qi = rint_i32((float)hq);
    const int sum = (int)((uint32_t)qi + (uint32_t)zi);
    return (uint32_t)clampi(sum, 0, kQmaxAsym8);
}
__device__ __forceinline__ int asym8_zero_int(float z) { return rint_i32((float)(f16)z); }

// ---------------------------------------------------------------------------------
// given-scale quantizer (asym_quant_host_8bit): 4 elements per lane step when the row
// length allows, else one
// ---------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void asym_quant8_kernel(const float *x, const float *scale, const float *zeros,
                                                          uint32_t rows, uint32_t cols, int8_t *q, bool vec)
{
    if (vec) {
        const uint32_t per_row = cols >> 2;
        const uint64_t total = (uint64_t)rows * per_row;
        for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (uint64_t)gridDim.x * blockDim.x) {
            const uint32_t row = (uint32_t)(i / per_row);
            const v4f32 v = __builtin_nontemporal_load(reinterpret_cast<const v4f32 *>(x) + i);
            const float s = scale[row];
            const int zi = asym8_zero_int(zeros[row]);
            uint32_t w = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) w |= asym8_code(v[e], s, zi) << (8 * e);
            reinterpret_cast<uint32_t *>(q)[i] = w;
        }
    } else {
        const uint64_t total = (uint64_t)rows * cols;
        for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (uint64_t)gridDim.x * blockDim.x) {
            const uint32_t row = (uint32_t)(i / cols);
            q[i] = (int8_t)asym8_code(x[i], scale[row], asym8_zero_int(zeros[row]));
        }
    }
}

int launch_asym_quant8(const float *x, const float *scale, const float *zeros, uint32_t rows, uint32_t cols, int8_t *q,
                       hipStream_t stream)
{
    if (rows == 0 || cols == 0) return 0;
    const bool vec = cols % 4 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(q) % 4 == 0;
    const uint64_t total = (uint64_t)rows * (vec ? cols / 4 : cols);
    const uint32_t blocks = (uint32_t)std::min<uint64_t>((total + 255) / 256, 1u << 20);
    hipLaunchKernelGGL(asym_quant8_kernel, dim3(blocks), dim3(256), 0, stream, x, scale, zeros, rows, cols, q, vec);
    return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------------
// fused row quantizer (AsymQuantizer8bit.forward in one pass): one workgroup per row, the row
// held in registers between the min / max reduction and the quantization (up to 8 x 4
// elements per lane; longer rows are read a second time, from L2)
// ---------------------------------------------------------------------------------
constexpr int kMaxVec8 = 8;

template <int WAVES, bool CACHED>
__global__ __launch_bounds__(WAVES * 64) void quantize_rows_asym8_kernel(const float *x, uint32_t rows, uint32_t cols,
                                                                         int8_t *q, float *scale, float *zeros)
{
    constexpr int T = WAVES * 64;
    __shared__ float red[2][WAVES];
    const uint32_t row = blockIdx.x, tid = threadIdx.x;
    const uint32_t nvec = cols >> 2;
    const v4f32 *xrow = reinterpret_cast<const v4f32 *>(x + (uint64_t)row * cols);
    uint32_t *qrow = reinterpret_cast<uint32_t *>(q + (uint64_t)row * cols);
    v4f32 regs[kMaxVec8];
    float lo = INFINITY, hi = -INFINITY;
    bool nan_seen = false;
    auto reduce = [&](const v4f32 &g) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            lo = fminf(lo, g[e]);
            hi = fmaxf(hi, g[e]);
            nan_seen |= g[e] != g[e];
        }
    };
    if (CACHED) {
#pragma unroll
        for (int i = 0; i < kMaxVec8; ++i) {
            const uint32_t u = tid + i * T;
            regs[i] = u < nvec ? __builtin_nontemporal_load(&xrow[u]) : v4f32{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int i = 0; i < kMaxVec8; ++i)
            if (tid + i * T < nvec) reduce(regs[i]);
    } else {
        for (uint32_t u = tid; u < nvec; u += T) reduce(xrow[u]);
    }
    lo = wave_min_f32(lo);
    hi = wave_max_f32(hi);
    nan_seen = __builtin_amdgcn_ballot_w64(nan_seen) != 0;
    if (WAVES > 1) {
        if ((tid & 63u) == 0) {
            red[0][tid >> 6] = nan_seen ? __builtin_nanf("") : lo;
            red[1][tid >> 6] = hi;
        }
        __syncthreads();
        lo = red[0][0];
        hi = red[1][0];
        nan_seen = lo != lo;
#pragma unroll
        for (int w = 1; w < WAVES; ++w) {
            nan_seen |= red[0][w] != red[0][w];
            lo = fminf(lo, red[0][w]);
            hi = fmaxf(hi, red[1][w]);
        }
    }
    if (nan_seen) lo = hi = __builtin_nanf("");  // torch's min / max return NaN for a row that holds one
    // scale = (max - min) / 127, zeros = round(-min / scale)  (quantizer.py:50-51), float32.  torch evaluates
    // tensor / scalar on a GPU as tensor * float32(1 / scalar), which is what the reference's scale is
    const float d = hi - lo;
    const float s = d * (1.0f / 127.0f);
    const float z = __builtin_rintf((-lo) / s);
    if (tid == 0) {
        scale[row] = s;
        zeros[row] = z;
    }
    const int zi = asym8_zero_int(z);
    auto quant4 = [&](const v4f32 &g) -> uint32_t {
        uint32_t w = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) w |= asym8_code(g[e], s, zi) << (8 * e);
        return w;
    };
    if (CACHED) {
#pragma unroll
        for (int i = 0; i < kMaxVec8; ++i) {
            const uint32_t u = tid + i * T;
            if (u < nvec) qrow[u] = quant4(regs[i]);
        }
    } else {
        for (uint32_t u = tid; u < nvec; u += T) qrow[u] = quant4(xrow[u]);
    }
}

int launch_quantize_rows_asym8(const float *x, uint32_t rows, uint32_t cols, int8_t *q, float *scale, float *zeros,
                               hipStream_t stream)
{
    if (rows == 0 || cols == 0) return 0;
    const uint32_t nvec = cols / 4;
    uint32_t waves = 1;
    while (waves < 16 && waves * 64 * 4 < nvec) waves *= 2;  // four 128-bit loads per lane when the row allows
    const bool cached = waves * 64 * kMaxVec8 >= nvec;
    const dim3 grid(rows);
#define DUQ_ROWS8(W)                                                                                              \
    case W:                                                                                                       \
        if (cached)                                                                                               \
            hipLaunchKernelGGL((quantize_rows_asym8_kernel<W, true>), grid, dim3(W * 64), 0, stream, x, rows, cols, q, scale, zeros); \
        else                                                                                                      \
            hipLaunchKernelGGL((quantize_rows_asym8_kernel<W, false>), grid, dim3(W * 64), 0, stream, x, rows, cols, q, scale, zeros); \
        break;
    switch (waves) {
        DUQ_ROWS8(1)
        DUQ_ROWS8(2)
        DUQ_ROWS8(4)
        DUQ_ROWS8(8)
        DUQ_ROWS8(16)
    }
#undef DUQ_ROWS8
    return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------------
// float32 dequant: x = (s_r * s_c) * (float(acc) - (z_r + z_c)) [+ bias]
// ---------------------------------------------------------------------------------
struct Epi8 {
    const float *s_row, *z_row, *s_col, *z_col, *bias;
};

__device__ __forceinline__ float dequant_hprec_one(int acc, float sr, float zr, float sc, float zc)
{
    const float scales = sr * sc;
    const float zeros = zr + zc;
    const float t = (float)acc - zeros;
    return scales * t;  // built with -ffp-contract=off: no fused multiply-add
}

__global__ __launch_bounds__(256) void dequant_hprec_kernel(const int32_t *acc, Epi8 e, uint32_t rows, uint32_t cols, float *x)
{
    const uint64_t total = (uint64_t)rows * cols;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (uint64_t)gridDim.x * blockDim.x) {
        const uint32_t row = (uint32_t)(i / cols), col = (uint32_t)(i % cols);
        float v = dequant_hprec_one(acc[i], e.s_row[row], e.z_row[row], e.s_col[col], e.z_col[col]);
        if (e.bias) v = v + e.bias[col];
        x[i] = v;
    }
}

int launch_dequant_hprec(const int32_t *acc, const float *s_row, const float *z_row, const float *s_col,
                         const float *z_col, const float *bias, uint32_t rows, uint32_t cols, float *x, hipStream_t stream)
{
    if (rows == 0 || cols == 0) return 0;
    const uint64_t total = (uint64_t)rows * cols;
    const uint32_t blocks = (uint32_t)std::min<uint64_t>((total + 255) / 256, 1u << 20);
    hipLaunchKernelGGL(dequant_hprec_kernel, dim3(blocks), dim3(256), 0, stream, acc, Epi8{s_row, z_row, s_col, z_col, bias},
                       rows, cols, x);
    return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------------
// GEMM  C[m,n] = sum_k A[m,k] * B[n,k]   (int8, int32 accumulation)
// ---------------------------------------------------------------------------------
// Tile 32*TM (M) x 256 (N), 4 wavefronts side by side along N (32*TM x 64 each, TM x 2 MFMA tiles of 32 x 32),
// 256-k chunks of 8 steps.  A wavefront's 64 weight rows are needed by no other wavefront, so weights go
// global -> registers: lane (r = lane % 32, h = lane / 32) holds bytes [32*s + 16*h, +16) of row r for step s, which
// is the operand layout of v_mfma_i32_32x32x32_i8; the register of step s is refetched for the next chunk as soon
// as the step's last MFMA has been issued, so every weight load has a whole chunk (64 MFMAs,
// 2048 cycles) to arrive.  Activations are shared by the four wavefronts: global -> registers -> LDS (three buffers, rows padded
// to 272 bytes, one barrier per chunk) -> fragments read one step ahead; the register of piece j is stored at step
// j (for the chunk after next) and refetched at once (for the chunk after that), again a whole chunk ahead.
// The weight operand is the MFMA "A" side, so a lane ends up with four consecutive output columns of one row.
// The first 56 bytes (through tiles_n) reach the kernels in registers (DUQ_HEAD_DECL / with_head).
struct Gemm8Params {
    const int8_t *A;  // [M, K]
    const int8_t *B;  // [N, K]
    uint32_t M, N, K;
    uint32_t tiles_m;
    int32_t *C;       // int32 out (not fused)
    float *y;         // float32 out (fused)
    uint32_t tiles_n;
    Epi8 epi;
};
static_assert(offsetof(Gemm8Params, epi) == kHeadBytes, "the fields delivered in registers");

__device__ __forceinline__ void lds_barrier8() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <int TM, int TN, bool FUSED, bool BIAS, bool TILED>
__global__ __launch_bounds__(256) void gemm_s8_kernel(DUQ_HEAD_DECL, Gemm8Params tail)
{
    Gemm8Params p = with_head(tail, DUQ_HEAD_USE);
    to_global(p.A);
    to_global(p.B);
    to_global(p.C);
    to_global(p.y);
    static_assert(TM == 8 || TM == 4 || TM == 2 || TM == 1, "32-row MFMA tiles per wavefront along M");
    // TN = 32-column MFMA tiles per wavefront: tiles of 256 columns (TN = 2), or of 128 (TN = 1, with 64-row tiles:
    // twice the workgroups for problems that leave CUs without a 64 x 256 tile)
    static_assert(TN == 2 || (TN == 1 && TM == 2), "column tiles per wavefront");
    constexpr int BM = 32 * TM, BN = 128 * TN;
    // steps (of 32 k) per chunk: 8, or 4 with 256-row tiles (TM = 8: all 256 accumulation registers hold accumulators
    // and three activation buffers of 256-k chunks would not fit in LDS)
    constexpr int NS = TM == 8 ? 4 : 8;
    constexpr uint32_t kChunk = 32 * NS;  // 256 (128)
    constexpr uint32_t kStride = kChunk + 16;
    constexpr uint32_t kBuf = BM * kStride;
    constexpr int PPR = kChunk / 16;      // 16-byte pieces per row of a chunk
    constexpr int NXP = BM * PPR / 256;   // 16-byte activation pieces per thread and chunk: 8, 4, 2 (TM = 8: 8)

    constexpr uint32_t kEStride = 32 * TN * 4 + 16;  // epilogue staging: 32 rows of 32*TN int32 per wavefront
    constexpr uint32_t kLds = 3 * kBuf > 4 * 32 * kEStride ? 3 * kBuf : 4 * 32 * kEStride;

    __shared__ __attribute__((aligned(16))) uint8_t lds[kLds];
    __shared__ float row_par[2][BM];  // the tile's per-row scale and zero point, fetched before the loop

    uint32_t tile_m, tile_n;
    tile_of_block(blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u, wave = tid >> 6;
    const uint32_t l32 = lane & 31u, h = lane >> 5;
    const uint32_t nchunks = (p.K + kChunk - 1) / kChunk;

    // tiled weights: whole 32-row tiles (the last one zero-padded), K * 32 bytes each
    const uint32_t wrows = TILED ? min((p.N + 31u) / 32u * 32u - n0, (uint32_t)BN) : min(p.N - n0, (uint32_t)BN);
    const __amdgpu_buffer_rsrc_t rW = make_rsrc(p.B + (uint64_t)n0 * p.K, wrows * p.K);
    const __amdgpu_buffer_rsrc_t rX = make_rsrc(p.A + (uint64_t)m0 * p.K, min(p.M - m0, (uint32_t)BM) * p.K);

    // K % 32 == 0, so a 16-byte piece is all inside a row or all past its end; pieces past K (in the last chunk, or of
    // chunks past the last) are redirected out of the descriptor's range and read as zero
    uint32_t wrow[TN];
#pragma unroll
    for (int t = 0; t < TN; ++t)
        wrow[t] = TILED ? (wave * (32 * TN) + t * 32) * p.K + lane * 16 : (wave * (32 * TN) + t * 32 + l32) * p.K + h * 16;
    auto load_w = [&](int t, int s, uint32_t c) -> v4i {
        const uint32_t k = c * kChunk + s * 32;  // + h*16 < K  <=>  k < K
        // tiled: the fragment of (tile, step) is 1 KB in lane order, steps one after the other
        return __builtin_bit_cast(v4i, buf_load16(rW, k < p.K ? wrow[t] + (TILED ? k * 32 : k) : kOobOffset, 0));
    };
    uint32_t xrow[NXP], xlds[NXP];
    const uint32_t xpiece = tid % PPR;
#pragma unroll
    for (int j = 0; j < NXP; ++j) {
        const uint32_t row = tid / PPR + j * (256 / PPR);
        xrow[j] = row * p.K + xpiece * 16;
        xlds[j] = row * kStride + xpiece * 16;
    }
    auto load_x = [&](int j, uint32_t c) -> v4u {
        const uint32_t k = c * kChunk;
        return buf_load16(rX, k + xpiece * 16 < p.K ? xrow[j] + k : kOobOffset, 0);
    };
    // fragment of rows b*32 + l32, step s: bytes [32*s + 16*h, +16) of the row's chunk
    const uint32_t frag = l32 * kStride + h * 16;
    auto read_x = [&](uint32_t buf, int b, int s) -> v4i {
        return *reinterpret_cast<const v4i *>(lds + buf + frag + b * 32 * kStride + s * 32);
    };

    constexpr int WR = 1;  // chunks of weights in flight (2 measured no faster: the loop is bound by bytes per cycle, not by latency)
    v4i wreg[WR][TN][NS];
    v4u xreg[NXP];
    v4i fx[2][TM];
    v16i32 acc[TN][TM];
#pragma unroll
    for (int t = 0; t < TN; ++t)
#pragma unroll
        for (int b = 0; b < TM; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[t][b][r] = 0;

    // ---- epilogue parameters first: their latency disappears behind the loop
    constexpr uint32_t kLanesPerRow = 8 * TN, kRowsPerStore = 64 / kLanesPerRow;  // a staged row is 128 * TN bytes
    const uint32_t c16 = lane % kLanesPerRow, r4 = lane / kLanesPerRow;
    const uint32_t n_out = n0 + wave * (32 * TN) + c16 * 4;  // first of the four output columns this lane stores
    float sc[4], zc[4], bs[4];
    if (FUSED) {
        if (tid < BM) {
            const uint32_t m = min(m0 + tid, p.M - 1);
            row_par[0][tid] = p.epi.s_row[m];
            row_par[1][tid] = p.epi.z_row[m];
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const uint32_t nn = min(n_out + r, p.N - 1);
            sc[r] = p.epi.s_col[nn];
            zc[r] = p.epi.z_col[nn];
            bs[r] = BIAS ? p.epi.bias[nn] : 0.f;
        }
    }

    // ---- prologue: activations of chunks 0 and 1 -> LDS, chunk 2 -> registers; weights of chunk 0
#pragma unroll
    for (int q = 0; q < 2; ++q) {
#pragma unroll
        for (int j = 0; j < NXP; ++j) xreg[j] = load_x(j, q);
#pragma unroll
        for (int j = 0; j < NXP; ++j) *reinterpret_cast<v4u *>(lds + q * kBuf + xlds[j]) = xreg[j];
    }
    // issued in the order of the main loop's chunks, so that the loop's wait counts are the same on entry and on
    // the back edge (the compiler takes the stricter of the two)
#pragma unroll
    for (int w = 0; w < WR; ++w) {
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            if (TM == 1) {
#pragma unroll
                for (int t = 0; t < TN; ++t) wreg[w][t][s] = load_w(t, s, w);
            }
            if (w == WR - 1) {
#pragma unroll
                for (int j = 0; j < NXP; ++j)
                    if (j * NS / NXP == s) xreg[j] = load_x(j, 2);
            }
            if (TM != 1) {
#pragma unroll
                for (int t = 0; t < TN; ++t) wreg[w][t][s] = load_w(t, s, w);
            }
        }
    }
    lds_barrier8();
#pragma unroll
    for (int b = 0; b < TM; ++b) fx[0][b] = read_x(0, b, 0);

    uint32_t cur = 0, nxt = kBuf, nx2 = 2 * kBuf;
    auto chunk = [&](auto par, uint32_t c) {
        constexpr int W = decltype(par)::value % WR;
#pragma unroll
        for (int s = 0; s < NS; ++s) {
#pragma unroll
            for (int b = 0; b < TM; ++b) {
#pragma unroll
                for (int t = 0; t < TN; ++t) {
                    asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0"
                                 : "+a"(acc[t][b])
                                 : "v"(wreg[W][t][s]), "v"(fx[s & 1][b]));
                    __builtin_amdgcn_sched_barrier(0);
                    // ---- side work in the shadow of this MFMA
                    if (t == 0)  // next step's fragment of this row tile (the next chunk's first step comes from `nxt`)
                        fx[(s + 1) & 1][b] = s + 1 < NS ? read_x(cur, b, s + 1) : read_x(nxt, b, 0);
                    if (b == TM - 1)  // last use of this step's weight register: refetch it for the next chunk
                        wreg[W][t][s] = load_w(t, s, c + WR);
                    // activation pieces: chunk c+2 -> its LDS buffer, then fetch chunk c+3; the pieces of a step in
                    // one slot, or (TM = 8: two pieces per step) in slots of their own
                    if (t == TN - 1 && (TM == 8 || b == 0)) {
#pragma unroll
                        for (int j = 0; j < NXP; ++j)
                            if (j * NS / NXP == s && (TM != 8 || b == 2 + 4 * (j % 2))) {
                                *reinterpret_cast<v4u *>(lds + nx2 + xlds[j]) = xreg[j];
                                xreg[j] = load_x(j, c + 3);
                            }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        // the MFMAs are opaque to the compiler's hazard tracking: accumulator copies at a join must find them retired
        asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
        lds_barrier8();
        const uint32_t t = cur;
        cur = nxt;
        nxt = nx2;
        nx2 = t;
    };
    using Even = std::integral_constant<int, 0>;
    using Odd = std::integral_constant<int, 1>;
    uint32_t c = 0;
    for (; c + 1 < nchunks; c += 2) {  // no branch inside the loop (the compiler's load counting stays exact)
        chunk(Even{}, c);
        chunk(Odd{}, c + 1);
    }
    if (c < nchunks) chunk(Even{}, c);
    asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");

    // ---- epilogue.  In the accumulators a lane holds row l32 and, for column tile t and q = 0..3, the four
    // consecutive columns 32*t + 8*q + 4*h + (0..3): stored from there, one instruction would touch 32 rows with 32
    // bytes each.  Each wavefront turns its 32 x 64 block around in its own piece of LDS (the loop's buffers are free
    // after the last barrier) so that a store instruction writes whole rows of 256 (128) contiguous bytes.
    uint8_t *stage = lds + wave * (32 * kEStride);
    const uint32_t n = n_out;
    const void *outp = FUSED ? (const void *)p.y : (const void *)p.C;
    const bool vec_ok = p.N % 4 == 0 && reinterpret_cast<uintptr_t>(outp) % 16 == 0;
#pragma unroll
    for (int b = 0; b < TM; ++b) {
#pragma unroll
        for (int t = 0; t < TN; ++t)
#pragma unroll
            for (int q = 0; q < 4; ++q)
                *reinterpret_cast<v4i *>(stage + l32 * kEStride + (t * 32 + q * 8 + h * 4) * 4) =
                    v4i{acc[t][b][q * 4], acc[t][b][q * 4 + 1], acc[t][b][q * 4 + 2], acc[t][b][q * 4 + 3]};
#pragma unroll
        for (int it = 0; it < 32 / (int)kRowsPerStore; ++it) {
            const uint32_t row = it * kRowsPerStore + r4;
            const v4i a = *reinterpret_cast<const v4i *>(stage + row * kEStride + c16 * 16);
            const uint32_t m = m0 + b * 32 + row;
            if (m >= p.M || n >= p.N) continue;
            if (FUSED) {
                const float sr = row_par[0][b * 32 + row], zr = row_par[1][b * 32 + row];
                v4f32 v;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float o = dequant_hprec_one(a[r], sr, zr, sc[r], zc[r]);
                    if (BIAS) o = o + bs[r];
                    v[r] = o;
                }
                float *dst = p.y + (uint64_t)m * p.N + n;
                if (vec_ok && n + 3 < p.N) {
                    __builtin_nontemporal_store(v, reinterpret_cast<v4f32 *>(dst));
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (n + r < p.N) dst[r] = v[r];
                }
            } else {
                int32_t *dst = p.C + (uint64_t)m * p.N + n;
                if (vec_ok && n + 3 < p.N) {
                    __builtin_nontemporal_store(a, reinterpret_cast<v4i *>(dst));
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (n + r < p.N) dst[r] = a[r];
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------
// skinny kernel (M <= 32): bound by reading the weight once from HBM
// ---------------------------------------------------------------------------------
// A workgroup owns 16 weight rows; its four wavefronts split K in contiguous quarters and meet in LDS at the end, so
// N / 16 workgroups fill the chip at decode sizes.  v_mfma_i32_16x16x64_i8 with the weights on the "A" side: lane
// (r = lane % 16, kb = lane / 16) holds 16 bytes of row r at k = 64*j + 16*kb for step j, from the row-major weight
// (16 rows x 64 contiguous bytes per load) or from the tiled copy (four runs of 256 contiguous bytes per load).  The
// activations (MT tiles of 16 rows) use the same layout on the "B" side, straight from global memory: they are
// small and stay in L2.  A ring of kSkinnyRing steps per operand is in flight per lane and each register is
// refetched right after its MFMA, so the whole K quarter of a 4096-long row is requested before the first MFMA.
constexpr int kSkinnyRing = 16;

template <int MT, bool FUSED, bool BIAS, bool TILED>
__global__ __launch_bounds__(256) void gemm_s8_skinny_kernel(DUQ_HEAD_DECL, Gemm8Params tail)
{
    Gemm8Params p = with_head(tail, DUQ_HEAD_USE);
    to_global(p.A);
    to_global(p.B);
    to_global(p.C);
    to_global(p.y);
    __shared__ v4i part[4][MT][64];
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u, wave = tid >> 6;
    const uint32_t l16 = lane & 15u, kb = lane >> 4;
    const uint32_t n0 = blockIdx.x * 16;
    const uint32_t steps = (p.K + 63) / 64;
    const uint32_t spw = (steps + 3) / 4;  // steps per wavefront
    const uint32_t j0 = wave * spw;

    // row-major: the descriptor covers this workgroup's rows (rows past N read as zero).  Tiled: it covers the 32-row
    // tile (zero-padded past N) of which these 16 rows are the lower or upper half
    const __amdgpu_buffer_rsrc_t rWt = TILED ? make_rsrc(p.B + (uint64_t)(n0 / 32) * 32 * p.K, 32u * p.K)
                                             : make_rsrc(p.B + (uint64_t)n0 * p.K, min(p.N - n0, 16u) * p.K);
    const __amdgpu_buffer_rsrc_t rX = make_rsrc(p.A, p.M * p.K);  // rows past M read as zero
    const bool wrow_ok = n0 + l16 < p.N;
    // byte offset of this lane's 16 bytes of step j: row-major  r*K + 64*j + 16*kb;
    // tiled (step ks = 2*j + kb/2, half h = kb%2, row r + 16*(n0/16 % 2) of the tile)  ks*1024 + (h*32 + row)*16
    const uint32_t wlane = TILED ? (kb >> 1) * 1024 + ((kb & 1u) * 32 + l16 + (n0 & 16u)) * 16 : l16 * p.K + kb * 16;
    auto load_w = [&](uint32_t j) -> v4i {
        const uint32_t k = j * 64 + kb * 16;
        const bool ok = wrow_ok && j < j0 + spw && k < p.K;
        return __builtin_bit_cast(v4i, buf_load16_aux<DUQ_S8_SKINNY_WLOAD_AUX>(rWt, ok ? wlane + (TILED ? j * 2048 : j * 64) : kOobOffset, 0));
    };
    auto load_x = [&](int mt, uint32_t j) -> v4i {
        const uint32_t k = j * 64 + kb * 16;
        const bool ok = j < j0 + spw && k < p.K;
        return __builtin_bit_cast(v4i, buf_load16(rX, ok ? (mt * 16 + l16) * p.K + k : kOobOffset, 0));
    };

    v4i w[kSkinnyRing], x[MT][kSkinnyRing];
#pragma unroll
    for (int u = 0; u < kSkinnyRing; ++u) {
        w[u] = load_w(j0 + u);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) x[mt][u] = load_x(mt, j0 + u);
    }
    v4i acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = v4i{0, 0, 0, 0};
    for (uint32_t g = 0; g < spw; g += kSkinnyRing) {
#pragma unroll
        for (int u = 0; u < kSkinnyRing; ++u) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[u], x[mt][u], acc[mt], 0, 0, 0);
            const uint32_t j = j0 + g + kSkinnyRing + u;  // past the wavefront's range: reads as zero
            w[u] = load_w(j);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) x[mt][u] = load_x(mt, j);
        }
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) part[wave][mt][lane] = acc[mt];
    __syncthreads();
    // lane (m = lane % 16, q = lane / 16) of tile mt holds C[mt*16 + m][n0 + 4*q + (0..3)]: MT * 64 threads finish
    if (tid >= MT * 64) return;
    const uint32_t mt = tid >> 6;
    v4i sum = part[0][mt][lane];
#pragma unroll
    for (int w2 = 1; w2 < 4; ++w2) {
        const v4i o = part[w2][mt][lane];
#pragma unroll
        for (int r = 0; r < 4; ++r) sum[r] += o[r];
    }
    const uint32_t m = mt * 16 + l16, n = n0 + kb * 4;
    if (m >= p.M || n >= p.N) return;
    const void *outp = FUSED ? (const void *)p.y : (const void *)p.C;
    const bool vec_ok = p.N % 4 == 0 && reinterpret_cast<uintptr_t>(outp) % 16 == 0 && n + 3 < p.N;
    if (FUSED) {
        const float sr = p.epi.s_row[m], zr = p.epi.z_row[m];
        v4f32 v;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const uint32_t nn = min(n + r, p.N - 1);
            float o = dequant_hprec_one(sum[r], sr, zr, p.epi.s_col[nn], p.epi.z_col[nn]);
            if (BIAS) o = o + p.epi.bias[nn];
            v[r] = o;
        }
        float *dst = p.y + (uint64_t)m * p.N + n;
        if (vec_ok) {
            *reinterpret_cast<v4f32 *>(dst) = v;
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (n + r < p.N) dst[r] = v[r];
        }
    } else {
        int32_t *dst = p.C + (uint64_t)m * p.N + n;
        if (vec_ok) {
            *reinterpret_cast<v4i *>(dst) = sum;
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (n + r < p.N) dst[r] = sum[r];
        }
    }
}

// ---------------------------------------------------------------------------------
// decode kernel (5 <= M <= 64 on the row-major weight): one round of workgroups, activations held in registers
// ---------------------------------------------------------------------------------
// The 4-bit MFMA decode kernel's shape for int8 (src/kernels/gemm.cu:46-81 at small M): eight wavefronts split K
// for one 16-column tile (wavefront v owns the 64-byte row segments [v*SEGS, (v+1)*SEGS)); lane (l16, g) holds
// bytes [g*16, +16) of each segment, of weight row l16 of the tile (MFMA "A" side) and of activation rows
// 16*t + l16 of the MT row tiles ("B" side), the operand layout of v_mfma_i32_16x16x64_i8.  A lane keeps its
// activation fragments in registers for the whole launch and a workgroup owns p.tiles_n consecutive column tiles
// with two tiles' weights in flight (two register sets alternate), so a launch is one round of at most 256
// workgroups and the activations (as many bytes as a tile's weights at 16 rows) enter a CU once.  The partial
// tiles meet in LDS; MT * 64 threads finish four consecutive columns of one row each.
template <int SEGS, int MT, bool FUSED, bool BIAS, bool TILED>
__global__ __launch_bounds__(512) void gemm_s8_decode_kernel(DUQ_HEAD_DECL, Gemm8Params tail)
{
    Gemm8Params p = with_head(tail, DUQ_HEAD_USE);
    to_global(p.A);
    to_global(p.B);
    to_global(p.C);
    to_global(p.y);
    constexpr int WAVES = 8;
    __shared__ v4i part[2][MT][WAVES][64];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t l16 = lane & 15u, g = lane >> 4;
    const uint32_t ntiles = (p.N + 15) / 16;
    const uint32_t tile0 = blockIdx.x * p.tiles_n;
    const uint32_t tile_end = min(tile0 + p.tiles_n, ntiles);

    // rows past N read as zero (the tiled copy holds whole 32-row tiles, zero-padded); N * K < 2^32 - 32 * K (launcher)
    const __amdgpu_buffer_rsrc_t rW = make_rsrc(p.B, (TILED ? (p.N + 31u) / 32u * 32u : p.N) * p.K);
    const __amdgpu_buffer_rsrc_t rX = make_rsrc(p.A, p.M * p.K);  // rows past M read as zero
    uint32_t koff[SEGS];  // byte offset inside a row, or out of range for pieces past K (K % 32 == 0 and 16 | off)
#pragma unroll
    for (int u = 0; u < SEGS; ++u) {
        const uint32_t off = (wave * SEGS + u) * 64 + g * 16;
        koff[u] = off < p.K ? off : kOobOffset;
    }
    // row-major: 16 rows x 64 contiguous bytes per load instruction.  Tiled copy (fragments of 32 rows x 32 bytes,
    // 1 KB each in lane order (r, h) -> (h * 32 + r) * 16): the 16 bytes of (row, 64 * j + 16 * g) sit in fragment
    // ks = 2 * j + g / 2 at lane (h = g % 2, r = row % 32): four runs of 256 contiguous bytes per instruction
    auto load_tile = [&](uint32_t tile, v4i(&w)[SEGS]) {
        const uint32_t row = tile * 16 + l16;
        const uint32_t nrows = tile < tile_end ? p.N : 0u;
        const uint32_t base = TILED ? (tile >> 1) * 32u * p.K + (g >> 1) * 1024u + ((g & 1u) * 32u + l16 + (tile & 1u) * 16u) * 16u
                                    : row * p.K;
#pragma unroll
        for (int u = 0; u < SEGS; ++u) {
            const uint32_t off = TILED ? base + (wave * SEGS + u) * 2048u : base + koff[u];
            w[u] = __builtin_bit_cast(v4i, buf_load16_aux<DUQ_S8_DEC_WLOAD_AUX>(rW, (row < nrows && koff[u] != kOobOffset) ? off : kOobOffset, 0));
        }
    };
    // loads in the order their data is needed: activations, the first tile's weights, the finishing threads' row
    // parameters
    v4i x[MT][SEGS];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int u = 0; u < SEGS; ++u)
            x[t][u] = __builtin_bit_cast(v4i, buf_load16(rX, koff[u] != kOobOffset ? (t * 16 + l16) * p.K + koff[u] : kOobOffset, 0));
    v4i w0[SEGS], w1[SEGS];
    load_tile(tile0, w0);

    // thread (mt = tid / 64, lane) finishes C[mt*16 + l16][tile*16 + 4*g + (0..3)]
    const bool finisher = tid < MT * 64;
    const uint32_t m = wave * 16 + l16;
    float sr = 0.f, zr = 0.f;
    if (FUSED && finisher) {
        const uint32_t mm = min(m, p.M - 1);
        sr = p.epi.s_row[mm], zr = p.epi.z_row[mm];
    }
    const void *outp = FUSED ? (const void *)p.y : (const void *)p.C;
    const bool vec_all = p.N % 4 == 0 && reinterpret_cast<uintptr_t>(outp) % 16 == 0;

    auto compute_tile = [&](uint32_t tile, const v4i(&w)[SEGS], uint32_t buf) {
        const uint32_t n = tile * 16 + g * 4;
        float sc[4], zc[4], bs[4];
        if (FUSED && finisher) {  // requested now, used after the matrix work and the barrier
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const uint32_t nn = min(n + r, p.N - 1);
                sc[r] = p.epi.s_col[nn];
                zc[r] = p.epi.z_col[nn];
                bs[r] = BIAS ? p.epi.bias[nn] : 0.f;
            }
        }
        v4i acc[MT];
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[t] = v4i{0, 0, 0, 0};
#pragma unroll
        for (int u = 0; u < SEGS; ++u)
#pragma unroll
            for (int t = 0; t < MT; ++t) acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[u], x[t][u], acc[t], 0, 0, 0);
#pragma unroll
        for (int t = 0; t < MT; ++t) part[buf][t][wave][lane] = acc[t];
        __syncthreads();
        if (finisher) {
            v4i sum = part[buf][wave][0][lane];
#pragma unroll
            for (int w2 = 1; w2 < WAVES; ++w2) {
                const v4i o = part[buf][wave][w2][lane];
#pragma unroll
                for (int r = 0; r < 4; ++r) sum[r] += o[r];
            }
            if (m < p.M && n < p.N) {
                const bool vec_ok = vec_all && n + 3 < p.N;
                if (FUSED) {
                    v4f32 v;
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        float o = dequant_hprec_one(sum[r], sr, zr, sc[r], zc[r]);
                        if (BIAS) o = o + bs[r];
                        v[r] = o;
                    }
                    float *dst = p.y + (uint64_t)m * p.N + n;
                    if (vec_ok) {
                        *reinterpret_cast<v4f32 *>(dst) = v;
                    } else {
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            if (n + r < p.N) dst[r] = v[r];
                    }
                } else {
                    int32_t *dst = p.C + (uint64_t)m * p.N + n;
                    if (vec_ok) {
                        *reinterpret_cast<v4i *>(dst) = sum;
                    } else {
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            if (n + r < p.N) dst[r] = sum[r];
                    }
                }
            }
        }
    };

    // the partial-sum buffers alternate with the register sets: one barrier per tile
    for (uint32_t t = tile0; t < tile_end; t += 2) {
        load_tile(t + 1, w1);
        compute_tile(t, w0, 0);
        load_tile(t + 2, w0);
        if (t + 1 < tile_end) compute_tile(t + 1, w1, 1);
    }
}

// shapes the decode kernel takes: up to 64 rows of at most 4096 elements (the activation fragments of more would
// not fit in registers next to two sets of weights; with 8192 it measured slower than the skinny kernel: 11.9
// against 10.5 us at 16 x 4096 x 8192), the weight tensor within 32-bit offsets; above 32 rows only up to 1024
// column tiles (64 rows, N = 28672: the 64-row tiles of the GEMM kernel take 27 us, this kernel 33).  Measured
// on the tiled copy, K = 4096, against the skinny kernel (64 rows: the GEMM kernel): N = 4096 M16 6.5 against
// 6.6 us, M32 7.7 against 8.9, M64 11.8 against 22.3; N = 11008 M16 11.1 against 14.7, M32 12.3 against 21.6, M64
// 17.3 against 24.9; N = 28672 M32 26.6 against 47.5; on the row-major weight it is 5-15 % slower than on the copy.
inline bool decode8_takes(uint32_t M, uint32_t N, uint32_t K)
{
    return M <= 64 && K <= 4096 && (M <= 32 || (N + 15) / 16 <= 1024) && ((uint64_t)N + 32) * K < 0xFFFFFF00ull;
}

template <bool FUSED, bool BIAS, bool TILED>
static void launch_decode8(Gemm8Params &p, hipStream_t stream)
{
    const uint32_t ntiles = (p.N + 15) / 16;
    p.tiles_n = (ntiles + 255) / 256;  // column tiles per workgroup: one round of at most 256 workgroups
    const dim3 grid((ntiles + p.tiles_n - 1) / p.tiles_n);
    const uint32_t mt = (p.M + 15) / 16;
#define DUQ_DEC8(S, T) DUQ_LAUNCH_HEAD((gemm_s8_decode_kernel<S, T, FUSED, BIAS, TILED>), grid, dim3(512), 0, stream, p)
    if (p.K > 2048) {
        if (mt == 1) DUQ_DEC8(8, 1);
        else if (mt == 2) DUQ_DEC8(8, 2);
        else if (mt == 3) DUQ_DEC8(8, 3);
        else DUQ_DEC8(8, 4);
    } else {
        if (mt == 1) DUQ_DEC8(4, 1);
        else if (mt == 2) DUQ_DEC8(4, 2);
        else if (mt == 3) DUQ_DEC8(4, 3);
        else DUQ_DEC8(4, 4);
    }
#undef DUQ_DEC8
}

// ---------------------------------------------------------------------------------
// rows kernel: M <= 4 activation rows on the row-major weight, rows of up to XS KB
// ---------------------------------------------------------------------------------
// The 4-bit rows kernel's shape for int8 (src/kernels/gemm.cu:46-81 at M <= 4): v_dot4_i32_i8 straight on the
// operands, a wavefront owns R weight rows and the whole K range (lane l holds bytes [i*1024 + l*16, +16) of each
// row: a load instruction covers 1 KB of one row and an activation register serves R rows), every weight load of
// the workgroup is requested before anything else, the MR * R partial sums of a lane meet the other lanes' through
// the wavefront's own piece of LDS (no barrier) and a few DPP steps.  A workgroup is four wavefronts: 16 (8 for rows
// longer than 4 KB) weight rows.
template <int MR, int XS, bool FUSED, bool BIAS>
__global__ __launch_bounds__(256) void gemv_s8_rows_kernel(DUQ_HEAD_DECL, Gemm8Params tail)
{
    Gemm8Params p = with_head(tail, DUQ_HEAD_USE);
    to_global(p.A);
    to_global(p.B);
    to_global(p.C);
    to_global(p.y);
    constexpr int R = XS <= 4 ? 4 : 2;  // weight rows per wavefront: at most 16 weight registers of 16 bytes per lane
    constexpr int V = MR * R;           // partial sums per lane: 2 .. 16
    constexpr int LPV = 64 / V;         // lanes that finish one sum
    static_assert((MR == 1 || MR == 2 || MR == 4) && MR * XS <= 16, "activation registers per lane");
    __shared__ __attribute__((aligned(16))) int red[4][V * 64];

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t n0 = (blockIdx.x * 4 + wave) * R;
    // loads in the order their data is needed: the activations, then every weight byte of this wavefront, then the
    // parameters of the output this lane will finish
    const __amdgpu_buffer_rsrc_t rX = make_rsrc(p.A, p.M * p.K);  // rows past M read as zero
    v4u xr[MR][XS];
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int i = 0; i < XS; ++i) {
            const uint32_t off = i * 1024 + lane * 16;
            xr[m][i] = buf_load16(rX, off < p.K ? m * p.K + off : kOobOffset, 0);  // K % 32 == 0 and 16 | off
        }
    const __amdgpu_buffer_rsrc_t rW = make_rsrc(p.B + (uint64_t)n0 * p.K, min(p.N - min(n0, p.N), (uint32_t)R) * p.K);
    v4u w[R][XS];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int i = 0; i < XS; ++i) {
            const uint32_t off = i * 1024 + lane * 16;
            w[r][i] = buf_load16_aux<DUQ_S8_ROWS_WLOAD_AUX>(rW, off < p.K ? r * p.K + off : kOobOffset, 0);  // rows past N: beyond the descriptor
        }
    const uint32_t myv = lane / LPV, sub = lane % LPV;
    const uint32_t my_m = myv / R, my_n = n0 + myv % R;
    float sr = 0.f, zr = 0.f, sc = 0.f, zc = 0.f, bias = 0.f;
    if (FUSED) {
        const uint32_t mm = min(my_m, p.M - 1), nn = min(my_n, p.N - 1);
        sr = p.epi.s_row[mm], zr = p.epi.z_row[mm], sc = p.epi.s_col[nn], zc = p.epi.z_col[nn];
        if (BIAS) bias = p.epi.bias[nn];
    }

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
                    acc[m][r] = __builtin_amdgcn_sdot4((int)w[r][i][d], (int)xr[m][i][d], acc[m][r], false);

    // the V sums of 64 lanes each: through this wavefront's piece of LDS (a wavefront's LDS operations execute in
    // order: no barrier), V entries per lane back, then log2(LPV) DPP steps
    int *mine = red[wave];
#pragma unroll
    for (int v = 0; v < V; ++v) mine[v * 64 + lane] = acc[v / R][v % R];
    __builtin_amdgcn_wave_barrier();
    int sum = 0;
#pragma unroll
    for (int e = 0; e < V; ++e) sum += mine[lane * V + e];  // = [myv * 64 + sub * V + e]
    // sum over the LPV consecutive lanes of a group (4 .. 32 lanes)
    sum += __builtin_amdgcn_update_dpp(0, sum, 0xB1, 0xF, 0xF, true);                  // quad_perm [1,0,3,2]
    sum += __builtin_amdgcn_update_dpp(0, sum, 0x4E, 0xF, 0xF, true);                  // quad_perm [2,3,0,1]
    if (LPV >= 8) sum += __builtin_amdgcn_update_dpp(0, sum, 0x141, 0xF, 0xF, true);   // row_half_mirror
    if (LPV >= 16) sum += __builtin_amdgcn_update_dpp(0, sum, 0x140, 0xF, 0xF, true);  // row_mirror
    if (LPV >= 32) sum += __shfl_xor(sum, 16, kWave);
    if (sub == 0 && my_m < p.M && my_n < p.N) {
        if (FUSED) {
            float o = dequant_hprec_one(sum, sr, zr, sc, zc);
            if (BIAS) o = o + bias;
            p.y[(uint64_t)my_m * p.N + my_n] = o;
        } else {
            p.C[(uint64_t)my_m * p.N + my_n] = sum;
        }
    }
}

template <int MR, bool FUSED, bool BIAS>
static void launch_rows8(const Gemm8Params &p, hipStream_t stream)
{
    const uint32_t xs = (p.K + 1023) / 1024;
#define DUQ_ROWS8K(XS)                                                                                              \
    DUQ_LAUNCH_HEAD((gemv_s8_rows_kernel<MR, XS, FUSED, BIAS>), dim3((p.N + 4 * (XS <= 4 ? 4 : 2) - 1) / (4 * (XS <= 4 ? 4 : 2))), \
                       dim3(256), 0, stream, p)
    if (xs <= 2) DUQ_ROWS8K(2);
    else if (xs <= 4) DUQ_ROWS8K(4);
    else if constexpr (MR <= 2) DUQ_ROWS8K(8);
#undef DUQ_ROWS8K
}

// shapes the rows kernel takes: row-major weight, up to four rows of at most 4096 elements (two rows: 8192), the
// weight tensor within 32-bit offsets per descriptor (a descriptor covers one wavefront's rows)
inline bool rows8_takes(uint32_t M, uint32_t K) { return M <= 4 && K <= (M <= 2 ? 8192u : 4096u); }

// a round of 256 x 256 tiles in rounds of 128 x 256 ones (measured 1.86 - 1.97: 4096 x 4096 x 4096 73.4 against
// 74.4 us, 4096 x 11008 x 4096 188 against 202, 4096 x 8192 x 8192 240 against 251)
#ifndef DUQ_S8_COST256
#define DUQ_S8_COST256 1.95f
#endif
template <bool FUSED, bool BIAS, bool TILED>
static void launch_gemm8_variant(Gemm8Params &p, hipStream_t stream)
{
    if (!TILED && rows8_takes(p.M, p.K)) {
        if (p.M == 1) launch_rows8<1, FUSED, BIAS>(p, stream);
        else if (p.M == 2) launch_rows8<2, FUSED, BIAS>(p, stream);
        else launch_rows8<4, FUSED, BIAS>(p, stream);
        return;
    }
    if (decode8_takes(p.M, p.N, p.K)) {
        launch_decode8<FUSED, BIAS, TILED>(p, stream);
        return;
    }
    if (p.M <= 32) {
        const dim3 grid((p.N + 15) / 16);
        if (p.M <= 16)
            DUQ_LAUNCH_HEAD((gemm_s8_skinny_kernel<1, FUSED, BIAS, TILED>), grid, dim3(256), 0, stream, p);
        else
            DUQ_LAUNCH_HEAD((gemm_s8_skinny_kernel<2, FUSED, BIAS, TILED>), grid, dim3(256), 0, stream, p);
        return;
    }
    p.tiles_n = (p.N + 255) / 256;
    // the tallest tile that still gives most of the 256 CUs a workgroup
    const uint32_t t128 = ((p.M + 127) / 128) * p.tiles_n, t64 = ((p.M + 63) / 64) * p.tiles_n;
    const uint32_t t256 = ((p.M + 255) / 256) * p.tiles_n;
    // 256-row tiles where every CU gets one and their rounds (each DUQ_S8_COST256 rounds of 128-row tiles for twice
    // the outputs) come out cheaper
    if (t256 >= 256 && DUQ_S8_COST256 * (float)((t256 + 255) / 256) < (float)((t128 + 255) / 256)) {
        p.tiles_m = (p.M + 255) / 256;
        DUQ_LAUNCH_HEAD((gemm_s8_kernel<8, 2, FUSED, BIAS, TILED>), dim3(p.tiles_m * p.tiles_n), dim3(256), 0, stream, p);
    } else if (p.M > 64 && t128 >= 160) {
        p.tiles_m = (p.M + 127) / 128;
        DUQ_LAUNCH_HEAD((gemm_s8_kernel<4, 2, FUSED, BIAS, TILED>), dim3(p.tiles_m * p.tiles_n), dim3(256), 0, stream, p);
    } else if (p.M > 32 && t64 >= 48) {
        p.tiles_m = (p.M + 63) / 64;
        // one round of 64 x 256 tiles would leave CUs idle: 64 x 128 tiles, twice as many (measured 21-24 % faster at
        // 128 such tiles, 9 % at 64)
        if (t64 <= 128) {
            p.tiles_n = (p.N + 127) / 128;
            DUQ_LAUNCH_HEAD((gemm_s8_kernel<2, 1, FUSED, BIAS, TILED>), dim3(p.tiles_m * p.tiles_n), dim3(256), 0, stream, p);
        } else {
            DUQ_LAUNCH_HEAD((gemm_s8_kernel<2, 2, FUSED, BIAS, TILED>), dim3(p.tiles_m * p.tiles_n), dim3(256), 0, stream, p);
        }
    } else {
        p.tiles_m = (p.M + 31) / 32;
        DUQ_LAUNCH_HEAD((gemm_s8_kernel<1, 2, FUSED, BIAS, TILED>), dim3(p.tiles_m * p.tiles_n), dim3(256), 0, stream, p);
    }
}

int launch_gemm_s8(const int8_t *A, const int8_t *B, bool b_tiled, uint32_t M, uint32_t N, uint32_t K, int32_t *C,
                   const float *s_row, const float *z_row, const float *s_col, const float *z_col, const float *bias,
                   float *y, hipStream_t stream)
{
    if (M == 0 || N == 0) return 0;
    Gemm8Params p{A, B, M, N, K, 0, C, y, 0, Epi8{s_row, z_row, s_col, z_col, bias}};
    if (C)
        launch_gemm8_variant<false, false, false>(p, stream);
    else if (b_tiled && bias)
        launch_gemm8_variant<true, true, true>(p, stream);
    else if (b_tiled)
        launch_gemm8_variant<true, false, true>(p, stream);
    else if (bias)
        launch_gemm8_variant<true, true, false>(p, stream);
    else
        launch_gemm8_variant<true, false, false>(p, stream);
    return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------------
// weight [N, K] row-major -> tiled: [ceil(N/32)][K/32][64 lanes][16 bytes], lane (r = lane % 32, h = lane / 32) of
// tile (nt, ks) holding W[32*nt + r][32*ks + 16*h, +16) (zero past row N): each MFMA weight fragment is then one
// contiguous kilobyte, eight cache lines per load instruction instead of thirty-two
// ---------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void weight_tile8_kernel(const int8_t *w, uint32_t N, uint32_t K, int8_t *out)
{
    const uint32_t ksteps = K / 32;
    const uint64_t pieces = (uint64_t)((N + 31) / 32) * ksteps * 64;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < pieces; i += (uint64_t)gridDim.x * blockDim.x) {
        const uint32_t ln = (uint32_t)(i & 63u);
        const uint64_t tile = i >> 6;
        const uint32_t ks = (uint32_t)(tile % ksteps), nt = (uint32_t)(tile / ksteps);
        const uint32_t row = nt * 32 + (ln & 31u), k = ks * 32 + (ln >> 5) * 16;
        v4u v = {0u, 0u, 0u, 0u};
        if (row < N) v = *reinterpret_cast<const v4u *>(w + (uint64_t)row * K + k);
        reinterpret_cast<v4u *>(out)[i] = v;
    }
}

int launch_weight_tile8(const int8_t *w, uint32_t N, uint32_t K, int8_t *out, hipStream_t stream)
{
    if (N == 0 || K == 0) return 0;
    const uint64_t pieces = (uint64_t)((N + 31) / 32) * (K / 32) * 64;
    const uint32_t blocks = (uint32_t)std::min<uint64_t>((pieces + 255) / 256, 1u << 20);
    hipLaunchKernelGGL(weight_tile8_kernel, dim3(blocks), dim3(256), 0, stream, w, N, K, out);
    return (int)hipGetLastError();
}

}  // namespace duq
