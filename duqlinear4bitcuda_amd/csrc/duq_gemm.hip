// Packed-int4 x packed-int4 -> int32 GEMM for gfx950 on v_mfma_i32_16x16x64_i8, with the
// fp16 dequant epilogue fused in (or raw int32 accumulators out).
//
//   C[m,n] = sum_k s4(A[m,k]) * s4(B[n,k])        (src/kernels/gemm.cu:8-43 of the reference)
//
// Nibble -> byte: for a packed word w, (w & 0xF0F0F0F0) holds the four odd-k nibbles as
// bytes equal to 16*s4 (sign included), ((w << 4) & 0xF0F0F0F0) the four even-k ones.
// Both operands are expanded the same way, so every MFMA product is 256*a*b and the
// accumulator is 256*C exactly; one arithmetic shift by 8 recovers C.  |C| <= 64*K, so
// 256*|C| stays below 2^31 for K <= 131008.  Integer accumulation is order-free, so the
// k order inside a tile only has to be the same for A and B.
//
// Six kernels here, picked by shape in select_gemm_kernel() (up to 64 rows run the two kernels of
// duq_decode.hip as far as they reach):
//  * stream kernel (prefill, more than 64 rows; tiles of 128, 64 or 32 rows x 256 columns or of 128 or 64 rows x
//    128, the shape picked per problem): weights go from global memory straight to registers, activations are
//    expanded once into LDS, v_mfma_i32_32x32x32_i8 with a hand-ordered schedule (see the kernel);
//  * short-row kernel (rows of at most 256 elements): the stream kernel's tile without its K pipeline;
//  * tile kernel (what is left, and any tensor of 4 GiB or more): BM x BN x 128 tiles, 4 wavefronts (2 x 2),
//    both operands expanded on the way into double-buffered LDS, v_mfma_i32_16x16x64_i8;
//  * ring kernel (17 <= M <= 256 on narrow problems or long rows, and 5..16 rows of 12289..16384 elements):
//    packed activations of all rows in LDS, every wavefront streams whole weight rows through a ring of loads;
//  * skinny kernel (9 <= M <= 16 with 1536 or more column tiles): one workgroup owns 16 output columns, its
//    wavefronts split K, whole-line weight loads turned into fragments through LDS;
//  * dot kernel (M <= 4 with rows longer than 16384 elements): v_dot8_i32_i4 on the packed nibbles, a
//    pure HBM stream.
// In the MFMA kernels the weight operand goes to the MFMA "A" side, so each lane ends up
// with four consecutive output columns of one row.
#include "duq_epilogue.h"
// Cache policy of the stream / short-row kernels' output stores: 2 = non-temporal (the output is written once and
// read by nobody in the launch; measured at M = 2048, N = K = 4096: 30.2 against 31.5 us, M = 4096: 58.8 against 61.1)
// Cache policy of the weight loads of the kernels that read every weight byte once: 2 = non-temporal.  Measured:
// skinny kernel 16 x 28672 x 4096 13.2 against 14.1 us, dot kernel 1 x 8192 x 28672 20.9 against 22.8 and 4 x 4096 x
// 20480 11.5 against 13.2; the ring kernel (row groups read the weights again; a lane fetches 16 bytes of a row, a
// quarter of a cache line, per instruction) loses on most shapes (100 x 1000 x 4096: 7.9 against 7.3) and keeps the
// default.
#ifndef DUQ_SKINNY_WLOAD_AUX
#define DUQ_SKINNY_WLOAD_AUX 2
#endif
#ifndef DUQ_RING_WLOAD_AUX
#define DUQ_RING_WLOAD_AUX 0
#endif
#ifndef DUQ_DOT_WLOAD_AUX
#define DUQ_DOT_WLOAD_AUX 2
#endif
#ifndef DUQ_STREAM_STORE_AUX
#define DUQ_STREAM_STORE_AUX 2
#endif
#include "duq_launch.h"
#include "duq_tiles.h"
#include <type_traits>

namespace duq {

constexpr uint32_t kNibbleMask = 0xF0F0F0F0u;

// The first 56 bytes (through tiles_n) reach the kernels in registers (DUQ_HEAD_DECL / with_head).
struct GemmParams {
    const uint8_t *A;  // activations [M, K/2]
    const uint8_t *B;  // weights     [N, K/2]
    uint32_t M, N, K;
    uint32_t tiles_m;
    int32_t *C;        // int32 out (EPI < 0)
    uint16_t *y;       // fp16 out  (EPI >= 0)
    uint32_t tiles_n;
    Epilogue epi;
};
static_assert(offsetof(GemmParams, epi) == kHeadBytes, "the fields delivered in registers");

// Batched launch: problem blockIdx.z of a batch whose tensors are contiguous ([batch, M, K/2], [batch, N, K/2],
// [batch, M, N], per-row arrays [batch, M], per-column arrays [batch, N]).
__device__ __forceinline__ void batch_shift(GemmParams &p, uint32_t b)
{
    p.A += (uint64_t)b * p.M * (p.K >> 1);
    p.B += (uint64_t)b * p.N * (p.K >> 1);
    if (p.C) p.C += (uint64_t)b * p.M * p.N;
    if (p.y) p.y += (uint64_t)b * p.M * p.N;
    batch_shift(p.epi, b, p.M, p.N);
}

__device__ __forceinline__ void expand_nibbles(const v4u w, v4u &even, v4u &odd)
{
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        even[i] = (w[i] << 4) & kNibbleMask;
        odd[i] = w[i] & kNibbleMask;
    }
}


// Store four consecutive output columns of one row.
template <int EPI, bool BIAS>
__device__ __forceinline__ void store_quad(const GemmParams &p, uint32_t m, uint32_t n0, v4i acc, bool vec_ok)
{
    if (m >= p.M || n0 >= p.N) return;
    if (EPI < 0) {
        int32_t *dst = p.C + (uint64_t)m * p.N + n0;
        if (vec_ok && n0 + 3 < p.N) {
            *reinterpret_cast<v4i *>(dst) = acc;
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (n0 + r < p.N) dst[r] = acc[r];
        }
    } else {
        constexpr int MODE = EPI < 0 ? 0 : EPI;
        const RowEpi rp = load_row<MODE>(p.epi, m);
        uint16_t out[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const uint32_t n = min(n0 + r, p.N - 1);
            const ColParams c = load_col<MODE, BIAS>(p.epi.s_col_1, p.epi.z_col_1, p.epi.s_col_2, p.epi.z_col_2,
                                                     p.epi.bias, n, p.epi.rs_col);
            out[r] = dequant_one<MODE, BIAS>(acc[r], rp, c);
        }
        uint16_t *dst = p.y + (uint64_t)m * p.N + n0;
        if (vec_ok && n0 + 3 < p.N) {
            *reinterpret_cast<v2u *>(dst) = v2u{(uint32_t)out[0] | ((uint32_t)out[1] << 16),
                                                (uint32_t)out[2] | ((uint32_t)out[3] << 16)};
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (n0 + r < p.N) dst[r] = out[r];
        }
    }
}

// ---------------------------------------------------------------------------------
// tile kernel
// ---------------------------------------------------------------------------------
constexpr int kBK = 128;           // k elements per tile step (64 packed bytes per row)
constexpr int kLdsStride = 144;    // bytes per LDS row: 128 expanded bytes + 16 pad

template <int BM, int BN, int EPI, bool BIAS>
__global__ __launch_bounds__(256) void gemm_s4_tile_kernel(DUQ_HEAD_DECL, GemmParams tail)
{
    GemmParams p = with_head(tail, DUQ_HEAD_USE);
    to_global(p.A);
    to_global(p.B);
    to_global(p.C);
    to_global(p.y);
    constexpr int WTM = BM / 2, WTN = BN / 2;  // per-wavefront tile
    constexpr int TM = WTM / 16, TN = WTN / 16;
    constexpr int NA = BM / 64, NB = BN / 64;  // 16-byte global pieces per thread
    static_assert(BM % 64 == 0 && BN % 64 == 0, "tile shape");

    __shared__ __attribute__((aligned(16))) uint8_t lds[2][(BM + BN) * kLdsStride];

    if (blockIdx.z) batch_shift(p, blockIdx.z);
    uint32_t tile_m, tile_n;
    tile_of_block(blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u, wave = tid >> 6;
    const uint32_t wm = wave >> 1, wn = wave & 1u;
    const uint32_t l16 = lane & 15u, g = lane >> 4;
    const uint32_t kbytes = p.K >> 1;
    const uint32_t nk = (p.K + kBK - 1) / kBK;

    // global source of each 16-byte piece this thread moves (row clamped to stay in bounds)
    const uint8_t *srcA[NA];
    const uint8_t *srcB[NB];
    uint32_t ldsA[NA], ldsB[NB];
    const uint32_t pj = tid & 3u;  // which 16-byte piece of the 64-byte row segment
#pragma unroll
    for (int i = 0; i < NA; ++i) {
        const uint32_t row = (tid >> 2) + i * 64;
        const uint32_t gm = min(m0 + row, p.M - 1);
        srcA[i] = p.A + (uint64_t)gm * kbytes + pj * 16;
        ldsA[i] = row * kLdsStride + pj * 32;
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
        const uint32_t row = (tid >> 2) + i * 64;
        const uint32_t gn = min(n0 + row, p.N - 1);
        srcB[i] = p.B + (uint64_t)gn * kbytes + pj * 16;
        ldsB[i] = (BM + row) * kLdsStride + pj * 32;
    }

    v4u ga[NA], gb[NB];
    auto load_tile = [&](uint32_t kt) {
        const uint32_t koff = kt * (kBK / 2);
        const bool ok = koff + pj * 16 < kbytes;  // K % 64 == 0: a piece is all in or all out
#pragma unroll
        for (int i = 0; i < NA; ++i)
            ga[i] = ok ? *reinterpret_cast<const v4u *>(srcA[i] + koff) : v4u{0u, 0u, 0u, 0u};
#pragma unroll
        for (int i = 0; i < NB; ++i)
            gb[i] = ok ? *reinterpret_cast<const v4u *>(srcB[i] + koff) : v4u{0u, 0u, 0u, 0u};
    };
    auto store_tile = [&](uint32_t buf) {
        uint8_t *base = lds[buf];
#pragma unroll
        for (int i = 0; i < NA; ++i) {
            v4u ev, od;
            expand_nibbles(ga[i], ev, od);
            *reinterpret_cast<v4u *>(base + ldsA[i]) = ev;
            *reinterpret_cast<v4u *>(base + ldsA[i] + 16) = od;
        }
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            v4u ev, od;
            expand_nibbles(gb[i], ev, od);
            *reinterpret_cast<v4u *>(base + ldsB[i]) = ev;
            *reinterpret_cast<v4u *>(base + ldsB[i] + 16) = od;
        }
    };

    v4i acc[TN][TM];
#pragma unroll
    for (int a = 0; a < TN; ++a)
#pragma unroll
        for (int b = 0; b < TM; ++b) acc[a][b] = v4i{0, 0, 0, 0};

    // fragment rows of this lane inside the LDS tile
    const uint32_t fragX = (wm * WTM + l16) * kLdsStride + g * 16;         // activations
    const uint32_t fragW = (BM + wn * WTN + l16) * kLdsStride + g * 16;    // weights

    load_tile(0);
    store_tile(0);
    __syncthreads();

    for (uint32_t kt = 0; kt < nk; ++kt) {
        const uint32_t cur = kt & 1u;
        const bool more = kt + 1 < nk;
        if (more) load_tile(kt + 1);

        const uint8_t *base = lds[cur];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            v4i fx[TM], fw[TN];
#pragma unroll
            for (int b = 0; b < TM; ++b)
                fx[b] = *reinterpret_cast<const v4i *>(base + fragX + b * 16 * kLdsStride + s * 64);
#pragma unroll
            for (int a = 0; a < TN; ++a)
                fw[a] = *reinterpret_cast<const v4i *>(base + fragW + a * 16 * kLdsStride + s * 64);
#pragma unroll
            for (int a = 0; a < TN; ++a)
#pragma unroll
                for (int b = 0; b < TM; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fw[a], fx[b], acc[a][b], 0, 0, 0);
        }

        if (more) store_tile(cur ^ 1u);
        __syncthreads();
    }

    // lane holds, for every (a, b): rows n = 4*g + r of the weight fragment, column m = l16
    const bool vec_ok = (EPI < 0) ? (p.N % 4 == 0 && reinterpret_cast<uintptr_t>(p.C) % 16 == 0)
                                  : (p.N % 4 == 0 && reinterpret_cast<uintptr_t>(p.y) % 8 == 0);
#pragma unroll
    for (int b = 0; b < TM; ++b)
#pragma unroll
        for (int a = 0; a < TN; ++a) {
            v4i v = acc[a][b];
#pragma unroll
            for (int r = 0; r < 4; ++r) v[r] >>= 8;
            store_quad<EPI, BIAS>(p, m0 + wm * WTM + b * 16 + l16, n0 + wn * WTN + a * 16 + g * 4, v, vec_ok);
        }
}

typedef int v16i __attribute__((ext_vector_type(16)));

// ---------------------------------------------------------------------------------
// stream kernel (prefill): weights global -> registers, activations through LDS,
// v_mfma_i32_32x32x32_i8
// ---------------------------------------------------------------------------------
// Tile 32*TM (M) x 256 (N), TM = 4 for large problems (described below; TM = 2 and 1 run the same
// schedule with 4 and 2 MFMA slots per step and exist to give mid-size M one workgroup per
// CU), 4 wavefronts side by side along N: every wavefront owns 64 weight
// rows that no other wavefront of the workgroup needs, so weight fragments never go through
// LDS: lane (l32, h) loads 16-byte piece i (0..3) = bytes [i*32 + h*16, +16) of the 128-byte
// row segment of a 256-k chunk straight into registers.  The 128 activation rows are shared
// by the four wavefronts: they are expanded to bytes once on the way into LDS (three
// buffers, rows padded to 272 B) and read back as 128-bit fragments.  LDS traffic per chunk
// is 32 KB written + 128 KB read.
//
// The 32x32x32 MFMA keeps the matrix pipe full from a single wavefront per SIMD (32 cycles
// per instruction, 16 per 32768 operations); the 16x16x64 form needs 18 and loses more to
// interleaved vector work.  A chunk is 8 k-steps (piece i, nibble parity) of 8 MFMAs (2
// weight tiles x 4 activation tiles).  The order is fixed by hand, a scheduling fence after
// every MFMA, and everything else rides in the MFMA shadows, a few instructions per slot:
//   every step    : the next step's four activation fragments (step 7: the next chunk's);
//   step 2i       : refetch weight piece i for the next chunk (its registers were just
//                   expanded), expand piece i+1 of weight tile 0;  step 2i+1: of tile 1;
//   step 1        : fetch the activations two chunks ahead;
//   steps 4..7    : expand + store those activations into the third LDS buffer;
//   steps 6, 7    : expand the next chunk's weight piece 0.
// MFMAs are issued through inline assembly with the accumulators tied to the accumulation
// register file, so they never move.
//
// All global reads are raw buffer loads on per-workgroup descriptors that cover exactly
// the rows of this tile: rows past M or N read as zero without a branch, and the chunk
// offset rides in the scalar offset.  The last chunks use per-piece guarded offsets (a
// piece at or past the row end is redirected out of bounds and reads as zero).
constexpr int kCK = 256;         // k elements per chunk (128 packed bytes per row)
constexpr int kXStride = 272;    // LDS bytes per activation row: 256 expanded + 16 pad


template <int TM, int EPI, bool BIAS, int TN = 2>
__global__ __launch_bounds__(256) void gemm_s4_stream_kernel(DUQ_HEAD_DECL, GemmParams tail)
{
    GemmParams p = with_head(tail, DUQ_HEAD_USE);
    to_global(p.A);
    to_global(p.B);
    to_global(p.C);
    to_global(p.y);
    static_assert(TM == 4 || TM == 2 || TM == 1, "32-row activation tiles per wavefront");
    // TN = 32-column weight tiles per wavefront: tiles of 256 columns (TN = 2), or of 128 with 64 rows (TN = 1):
    // as many outputs per workgroup as 32 x 256 with a third less operand bytes into the CU
    static_assert(TN == 2 || (TN == 1 && TM >= 2), "column tiles per wavefront");
    constexpr int BM = 32 * TM, BN = 128 * TN;
    constexpr int S = TM * TN;         // MFMA slots per step
    constexpr int NXP = TM;            // 16-byte activation pieces per thread and chunk
    constexpr uint32_t kBuf = BM * kXStride;

    __shared__ __attribute__((aligned(16))) uint8_t lds[3 * kBuf];
    // dual-uniform row-sum epilogue (EPI 5): its parameters, eight words per column of the tile and per row,
    // fetched by the first BN / BM threads before the loop and read back from here after it
    //   column: wlo, whi (first eight bytes of the weight row), s1 | s2 << 16, z1, z2, adj1, adj2, bias
    //   row   : xlo, xhi & 0xFF (first ten codes of the activation row), float(s), z, rx - rxl, rxl
    __shared__ __attribute__((aligned(16))) uint32_t dpar[EPI == 5 ? (BN + BM) * 8 : 4];
    __shared__ uint32_t dwide;  // EPI 5: non-zero when a factor of the corrections leaves the signed 24-bit range

    if (blockIdx.z) batch_shift(p, blockIdx.z);
    uint32_t tile_m, tile_n;
    tile_of_block(blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u, wave = tid >> 6;
    const uint32_t l32 = lane & 31u, h = lane >> 5;
    const uint32_t kbytes = p.K >> 1;
    const uint32_t nfull = p.K / kCK;
    const uint32_t nchunks = (p.K + kCK - 1) / kCK;

    if constexpr (EPI == 5) {
        if (tid == 0) dwide = 0;
        __syncthreads();
        bool wide = false;
        if (tid < (uint32_t)BN) {
            const uint32_t n = min(n0 + tid, p.N - 1);
            const v2u head = *reinterpret_cast<const v2u *>(p.B + (uint64_t)n * kbytes);
            uint32_t *d = dpar + tid * 8;
            d[0] = head[0];
            d[1] = head[1];
            d[2] = (uint32_t)p.epi.s_col_1[n] | ((uint32_t)p.epi.s_col_2[n] << 16);
            d[3] = (uint32_t)rint_i32((float)bits_to_f16(p.epi.z_col_1[n]));
            d[4] = (uint32_t)rint_i32((float)bits_to_f16(p.epi.z_col_2[n]));
            d[5] = (uint32_t)p.epi.rs_col[n];
            d[6] = (uint32_t)p.epi.rs_col_2[n];
            d[7] = BIAS ? (uint32_t)p.epi.bias[n] : 0u;
            wide = !(fits_i24(d[3]) && fits_i24(d[4]) && fits_i24(d[5]) && fits_i24(d[6]));
        }
        if (tid < (uint32_t)BM) {
            const uint32_t m = min(m0 + tid, p.M - 1);
            const v2u head = *reinterpret_cast<const v2u *>(p.A + (uint64_t)m * kbytes);
            const uint32_t xlo = head[0], xhi = head[1] & 0xFFu;  // input columns 0..7 and 8, 9
            const uint32_t rxl = (uint32_t)__builtin_amdgcn_sdot8((int)xhi, 0x11111111, __builtin_amdgcn_sdot8((int)xlo, 0x11111111, 0, false), false);
            uint32_t *d = dpar + (BN + tid) * 8;
            d[0] = xlo;
            d[1] = xhi;
            d[2] = __builtin_bit_cast(uint32_t, (float)bits_to_f16(p.epi.s_row[m]));
            d[3] = (uint32_t)rint_i32((float)bits_to_f16(p.epi.z_row[m]));
            d[4] = (uint32_t)p.epi.rs_row[m] - rxl;
            d[5] = rxl;
            wide = wide || !(fits_i24(d[3]) && fits_i24(d[4]));
        }
        if (wide) dwide = 1;  // (same value from every writer)
        // (the barrier that ends the prologue below orders these writes before the epilogue's reads)
    }

    const __amdgpu_buffer_rsrc_t rW = make_rsrc(p.B + (uint64_t)n0 * kbytes, min(p.N - n0, (uint32_t)BN) * kbytes);
    const __amdgpu_buffer_rsrc_t rX = make_rsrc(p.A + (uint64_t)m0 * kbytes, min(p.M - m0, (uint32_t)BM) * kbytes);

    uint32_t woff[TN];
#pragma unroll
    for (int t = 0; t < TN; ++t) woff[t] = (wave * (32 * TN) + t * 32 + l32) * kbytes + h * 16;
    uint32_t xoff[NXP], xlds[NXP];
    const uint32_t xq = tid & 7u;  // which 16-byte piece of the 128-byte row segment
#pragma unroll
    for (int i = 0; i < NXP; ++i) {
        const uint32_t row = (tid >> 3) + i * 32;
        xoff[i] = row * kbytes + xq * 16;
        xlds[i] = row * kXStride + xq * 32;
    }

    v4u wreg[TN][4];      // raw weight pieces [tile][piece]
    v4u xreg[NXP];        // raw activation pieces
    v4u wexp[2][2][TN];   // expanded weights [piece & 1][parity][tile]
    v4i fx[2][TM];        // activation fragments [step & 1][tile]
    v16i acc[TN][TM];
#pragma unroll
    for (int t = 0; t < TN; ++t)
#pragma unroll
        for (int b = 0; b < TM; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[t][b][r] = 0;

    // fragment of step (i, par) for activation tile b: + b*32*kXStride + i*64 + par*16
    const uint32_t fragX = l32 * kXStride + h * 32;

    auto expand_word = [&](const v4u &raw, v4u &even, v4u &odd, int w) {
        even[w] = (raw[w] << 4) & kNibbleMask;
        odd[w] = raw[w] & kNibbleMask;
    };

    // GUARD = false: every chunk fetched is complete, plain offsets.
    auto body = [&](auto guard, uint32_t c, uint32_t cur, uint32_t nxt, uint32_t nx2) {
        constexpr bool G = decltype(guard)::value;
        const uint32_t koff1 = (c + 1) * (kCK / 2), koff2 = (c + 2) * (kCK / 2);
        const bool okx = !G || (koff2 + xq * 16 < kbytes);  // K % 64 == 0: a piece is all in or all out
        v4u xe, xo;
#pragma unroll
        for (int step = 0; step < 8; ++step) {
            const int i = step >> 1, par = step & 1;
            const bool okw = !G || (koff1 + i * 32 + h * 16 < kbytes);
#pragma unroll
            for (int slot = 0; slot < S; ++slot) {
                const int b = slot / TN, t = slot % TN;
                asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0"
                             : "+a"(acc[t][b])
                             : "v"(wexp[i & 1][par][t]), "v"(fx[step & 1][b]));
                __builtin_amdgcn_sched_barrier(0);
                // ---- side work in the shadow of this MFMA
                if (slot < TM) {  // next step's activation fragment for tile `slot`
                    const uint8_t *src = step < 7 ? lds + cur + fragX + ((step + 1) >> 1) * 64 + ((step + 1) & 1) * 16
                                                  : lds + nxt + fragX;
                    fx[(step + 1) & 1][slot] = *reinterpret_cast<const v4i *>(src + slot * 32 * kXStride);
                }
                if (par == 0 && slot < TN)  // piece i was expanded earlier: refetch it for the next chunk
                    wreg[slot][i] = buf_load16(rW, okw ? woff[slot] + i * 32 : kOobOffset, koff1);
                if (step == 1 && slot < NXP)  // activations two chunks ahead
                    xreg[slot] = buf_load16(rX, okx ? xoff[slot] : kOobOffset, koff2);
                // expand the next weight piece of tile `par`: its four words over the last four slots (or
                // two / one per slot when a step has fewer than four slots)
                if (par < TN) {
                    const int np = (i + 1) & 3;  // pieces 1, 2, 3 of this chunk, then piece 0 of the next
#pragma unroll
                    for (int w = 0; w < 4; ++w)
                        if ((S >= 4 ? S - 4 + w : w * S / 4) == slot)
                            expand_word(wreg[par < TN ? par : 0][np], wexp[(i + 1) & 1][0][par < TN ? par : 0],
                                        wexp[(i + 1) & 1][1][par < TN ? par : 0], w);
                }
                if (step >= 8 - NXP) {  // activations two chunks ahead -> third LDS buffer, one piece per step
#pragma unroll
                    for (int w = 0; w < 4; ++w)
                        if ((S >= 4 ? w : w * S / 4) == slot) {
                            expand_word(xreg[step - (8 - NXP)], xe, xo, w);
                            if (w == 3) {
                                *reinterpret_cast<v4u *>(lds + nx2 + xlds[step - (8 - NXP)]) = xe;
                                *reinterpret_cast<v4u *>(lds + nx2 + xlds[step - (8 - NXP)] + 16) = xo;
                            }
                        }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        __syncthreads();
    };

    using Plain = std::false_type;
    using Guarded = std::true_type;

    // ---- prologue: chunks 0 and 1 activations -> LDS, chunk 0 weights -> registers
    {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const bool okw = i * 32 + h * 16 < kbytes;
#pragma unroll
            for (int t = 0; t < TN; ++t) wreg[t][i] = buf_load16(rW, okw ? woff[t] + i * 32 : kOobOffset, 0);
        }
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const bool okx = q * (kCK / 2) + xq * 16 < kbytes;
#pragma unroll
            for (int i = 0; i < NXP; ++i) xreg[i] = buf_load16(rX, okx ? xoff[i] : kOobOffset, q * (kCK / 2));
#pragma unroll
            for (int i = 0; i < NXP; ++i) {
                v4u ev, od;
                expand_nibbles(xreg[i], ev, od);
                *reinterpret_cast<v4u *>(lds + q * kBuf + xlds[i]) = ev;
                *reinterpret_cast<v4u *>(lds + q * kBuf + xlds[i] + 16) = od;
            }
        }
#pragma unroll
        for (int t = 0; t < TN; ++t) expand_nibbles(wreg[t][0], wexp[0][0][t], wexp[0][1][t]);
        __syncthreads();
#pragma unroll
        for (int b = 0; b < TM; ++b) fx[0][b] = *reinterpret_cast<const v4i *>(lds + fragX + b * 32 * kXStride);
    }

    // ---- epilogue parameters: fetched now so that their latency hides behind the main loop
#include "duq_stream_epilogue_fetch.inc"

    uint32_t cur = 0, nxt = kBuf, nx2 = 2 * kBuf;
    auto rotate = [&]() {
        const uint32_t t = cur;
        cur = nxt;
        nxt = nx2;
        nx2 = t;
    };
    uint32_t c = 0;
    for (; c + 2 < nfull; ++c) {  // steady state: chunks c+1 and c+2 are complete ones
        body(Plain{}, c, cur, nxt, nx2);
        rotate();
    }
    for (; c < nchunks; ++c) {  // last chunks: guarded fetches (a fetch past K reads zeros, unused)
        body(Guarded{}, c, cur, nxt, nx2);
        rotate();
    }
    // the MFMAs above are opaque to the compiler's hazard tracking: let the last ones retire
    // before the accumulators are read
    asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");

    constexpr bool kWideStore = false;
#include "duq_stream_epilogue_store.inc"
}

// ---------------------------------------------------------------------------------
// stream kernel, 256-row tiles: problems with at least one 256 x 256 tile per CU
// ---------------------------------------------------------------------------------
// The stream kernel's schedule with twice the activation rows per workgroup: the weight bytes a wavefront fetches
// and expands (the loop's main side work: two vector instructions per packed word) meet eight activation tiles
// instead of four, and a tile's prologue and epilogue are paid once per 65536 outputs instead of twice.  All 256
// accumulation registers hold accumulators (2 weight tiles x 8 activation tiles x 16), so the epilogue parameters
// are fetched after the loop, and a chunk is 128 k (three LDS buffers of 256 rows x 144 bytes; the epilogue's staging
// area, 4 x 256 x 144 bytes, is what sizes the array).  A chunk is four steps (piece, nibble parity) of sixteen
// MFMAs; per step: slots 0-7 read the next step's eight activation fragments, 8-9 refetch the weight piece just
// consumed (even steps), 10-13 expand one weight piece of one tile, 8, 9, 14, 15 expand one activation piece (stored
// in slot 15), and the activations ride two chunks of registers deep: a chunk's packed activations are requested a
// whole chunk before they are expanded into the buffer that is read two chunks later.
constexpr int kCK2 = 128;        // k elements per chunk
constexpr int kXStride2 = 144;   // LDS bytes per activation row: 128 expanded + 16 pad

template <int EPI, bool BIAS>
__global__ __launch_bounds__(256) void gemm_s4_stream256_kernel(DUQ_HEAD_DECL, GemmParams tail)
{
    GemmParams p = with_head(tail, DUQ_HEAD_USE);
    to_global(p.A);
    to_global(p.B);
    to_global(p.C);
    to_global(p.y);
    static_assert(EPI != 5, "the dual-uniform row-sum epilogue stages its parameters in LDS: stream kernel");
    constexpr int TM = 8, TN = 2, BM = 256, BN = 256, S = TM * TN, NXP = 4;
    constexpr uint32_t kBuf = BM * kXStride2;
    constexpr uint32_t kLds = 4 * BM * 144 > 3 * kBuf ? 4 * BM * 144 : 3 * kBuf;
    __shared__ __attribute__((aligned(16))) uint8_t lds[kLds];
    uint32_t *const dpar = nullptr;  // named by the shared epilogue text for an epilogue this kernel never runs
    const uint32_t dwide = 0;

    if (blockIdx.z) batch_shift(p, blockIdx.z);
    uint32_t tile_m, tile_n;
    tile_of_block(blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u, wave = tid >> 6;
    const uint32_t l32 = lane & 31u, h = lane >> 5;
    const uint32_t kbytes = p.K >> 1;
    const uint32_t nchunks = (p.K + kCK2 - 1) / kCK2;

    const __amdgpu_buffer_rsrc_t rW = make_rsrc(p.B + (uint64_t)n0 * kbytes, min(p.N - n0, (uint32_t)BN) * kbytes);
    const __amdgpu_buffer_rsrc_t rX = make_rsrc(p.A + (uint64_t)m0 * kbytes, min(p.M - m0, (uint32_t)BM) * kbytes);

    // weights: lane (l32, h) of tile t holds piece i = bytes [i*32 + h*16, +16) of the chunk's 64-byte row segment
    uint32_t woff[TN];
#pragma unroll
    for (int t = 0; t < TN; ++t) woff[t] = (wave * (32 * TN) + t * 32 + l32) * kbytes + h * 16;
    // activations: thread -> 16-byte piece xq of the segment of row xrow + 64 * i.  The sixteen lanes that an LDS
    // write instruction serves together hold rows r, r + 1, r + 8, r + 9 (r even): with 144-byte rows their four
    // pieces each land in sixteen different 16-byte columns of the banks (rows r .. r + 3 would collide in pairs)
    uint32_t xoff[NXP], xlds[NXP];
    const uint32_t xq = tid & 3u;
    const uint32_t xrow = ((tid >> 2) & 1u) + 8u * ((tid >> 3) & 1u) + 2u * ((tid >> 4) & 3u) + 16u * (tid >> 6);
#pragma unroll
    for (int i = 0; i < NXP; ++i) {
        const uint32_t row = xrow + i * 64;
        xoff[i] = row * kbytes + xq * 16;
        xlds[i] = row * kXStride2 + xq * 32;
    }
    // K % 64 == 0: a 16-byte piece is all inside the row or all outside (then redirected out of range: zero)
    auto load_w = [&](int t, int i, uint32_t koff) {
        return buf_load16(rW, koff + i * 32 + h * 16 < kbytes ? woff[t] + i * 32 : kOobOffset, koff);
    };
    auto load_x = [&](int j, uint32_t koff) {
        return buf_load16(rX, koff + xq * 16 < kbytes ? xoff[j] : kOobOffset, koff);
    };

    v4u wreg[TN][2];      // raw weight pieces [tile][piece]
    v4u xr[2][NXP];       // raw activation pieces, two chunks of them
    v4u wexp[2][2][TN];   // expanded weights [piece][parity][tile]
    v4i fx[2][TM];        // activation fragments [step & 1][tile]
    v16i acc[TN][TM];
#pragma unroll
    for (int t = 0; t < TN; ++t)
#pragma unroll
        for (int b = 0; b < TM; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[t][b][r] = 0;

    // fragment of step (i, par) for activation tile b: + b*32*kXStride2 + i*64 + par*16
    const uint32_t fragX = l32 * kXStride2 + h * 32;
    auto expand_word = [&](const v4u &raw, v4u &even, v4u &odd, int w) {
        even[w] = (raw[w] << 4) & kNibbleMask;
        odd[w] = raw[w] & kNibbleMask;
    };

    // chunk c; PAR = c & 1: xr[PAR] holds the packed activations of chunk c + 2, xr[PAR ^ 1] receives those of c + 3
    auto body = [&](auto parity, uint32_t c, uint32_t cur, uint32_t nxt, uint32_t nx2) {
        constexpr int PAR = decltype(parity)::value;
        const uint32_t koff1 = (c + 1) * (kCK2 / 2), koff3 = (c + 3) * (kCK2 / 2);
        v4u xe, xo;
#pragma unroll
        for (int step = 0; step < 4; ++step) {
            const int i = step >> 1, par = step & 1;
#pragma unroll
            for (int slot = 0; slot < S; ++slot) {
                const int b = slot / TN, t = slot % TN;
                asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0"
                             : "+a"(acc[t][b])
                             : "v"(wexp[i][par][t]), "v"(fx[step & 1][b]));
                __builtin_amdgcn_sched_barrier(0);
                // ---- side work in the shadow of this MFMA
                if (slot < TM) {  // next step's activation fragment for tile `slot`
                    const uint8_t *src = step < 3 ? lds + cur + fragX + ((step + 1) >> 1) * 64 + ((step + 1) & 1) * 16
                                                  : lds + nxt + fragX;
                    fx[(step + 1) & 1][slot] = *reinterpret_cast<const v4i *>(src + slot * 32 * kXStride2);
                }
                if (par == 0 && slot >= 8 && slot < 8 + TN)  // piece i was expanded earlier: refetch it for the next chunk
                    wreg[slot - 8][i] = load_w(slot - 8, i, koff1);
                if (slot >= 10 && slot < 14)  // the next piece (this chunk's second, then the next chunk's first) of tile `par`
                    expand_word(wreg[par][(i + 1) & 1], wexp[(i + 1) & 1][0][par], wexp[(i + 1) & 1][1][par], slot - 10);
                if (step == 0 && slot >= 12) xr[PAR ^ 1][slot - 12] = load_x(slot - 12, koff3);
                // chunk c + 2 -> third LDS buffer: piece `step`, its four words in the slots without a fragment read
                // or a weight word, then both halves stored
                if (slot == 8 || slot == 9 || slot == 14 || slot == 15) {
                    const int w = slot < 10 ? slot - 8 : slot - 12;
                    expand_word(xr[PAR][step], xe, xo, w);
                    if (w == 3) {
                        *reinterpret_cast<v4u *>(lds + nx2 + xlds[step]) = xe;
                        *reinterpret_cast<v4u *>(lds + nx2 + xlds[step] + 16) = xo;
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        __syncthreads();
    };

    // ---- prologue: chunks 0 and 1 activations -> LDS, chunk 2 -> registers, chunk 0 weights -> registers
    {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int t = 0; t < TN; ++t) wreg[t][i] = load_w(t, i, 0);
#pragma unroll
        for (int q = 0; q < 2; ++q) {
#pragma unroll
            for (int j = 0; j < NXP; ++j) xr[q][j] = load_x(j, q * (kCK2 / 2));
        }
#pragma unroll
        for (int q = 0; q < 2; ++q)
#pragma unroll
            for (int j = 0; j < NXP; ++j) {
                v4u ev, od;
                expand_nibbles(xr[q][j], ev, od);
                *reinterpret_cast<v4u *>(lds + q * kBuf + xlds[j]) = ev;
                *reinterpret_cast<v4u *>(lds + q * kBuf + xlds[j] + 16) = od;
            }
#pragma unroll
        for (int j = 0; j < NXP; ++j) xr[0][j] = load_x(j, 2 * (kCK2 / 2));
#pragma unroll
        for (int t = 0; t < TN; ++t) expand_nibbles(wreg[t][0], wexp[0][0][t], wexp[0][1][t]);
        __syncthreads();
#pragma unroll
        for (int b = 0; b < TM; ++b) fx[0][b] = *reinterpret_cast<const v4i *>(lds + fragX + b * 32 * kXStride2);
    }

    uint32_t cur = 0, nxt = kBuf, nx2 = 2 * kBuf;
    auto rotate = [&]() {
        const uint32_t t = cur;
        cur = nxt;
        nxt = nx2;
        nx2 = t;
    };
    using P0 = std::integral_constant<int, 0>;
    using P1 = std::integral_constant<int, 1>;
    uint32_t c = 0;
    for (; c + 1 < nchunks; c += 2) {
        body(P0{}, c, cur, nxt, nx2);
        rotate();
        body(P1{}, c + 1, cur, nxt, nx2);
        rotate();
    }
    if (c < nchunks) body(P0{}, c, cur, nxt, nx2);
    // the MFMAs above are opaque to the compiler's hazard tracking: let the last ones retire
    // before the accumulators are read
    asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");

    // ---- epilogue parameters (after the loop: no registers to spare inside it), then the epilogue
#include "duq_stream_epilogue_fetch.inc"
    constexpr bool kWideStore = false;
#include "duq_stream_epilogue_store.inc"
}

// ---------------------------------------------------------------------------------
// short-row kernel: K <= 256 (one chunk), many tiles; batched products of short rows
// ---------------------------------------------------------------------------------
// The stream kernel's tile (32*TM rows x 256 columns, four wavefronts side by side along N, weights global ->
// registers, activations expanded into LDS, v_mfma_i32_32x32x32_i8, the same epilogue) without its K pipeline: a
// problem whose rows hold at most 256 elements is one chunk, and a launch is its output stores (a 2048 x 2048 x 128
// product moves 0.5 MB in and 8 MB out).  One activation buffer that doubles as the epilogue's staging area (37 KB
// of LDS at 64 rows), only the steps the row length needs, whole-row stores; two workgroups share a CU (about 200
// registers each) and overlap one another's loads, matrix work and stores.  (Persistent workgroups that request
// the next tile's operands before the current tile's epilogue measured slower, 93 against 86 us on 32 products of
// 2048 x 2048 x 128: the loop-carried wait for those loads also waits for the stores issued after them.)
template <int TM, int EPI, bool BIAS>
__global__ __launch_bounds__(256, 2) void gemm_s4_shortk_kernel(DUQ_HEAD_DECL, GemmParams tail)
{
    GemmParams p = with_head(tail, DUQ_HEAD_USE);
    to_global(p.A);
    to_global(p.B);
    to_global(p.C);
    to_global(p.y);
    constexpr int BM = 32 * TM, BN = 256, TN = 2;
    constexpr int NXP = TM;  // 16-byte activation pieces per thread
    constexpr uint32_t kBuf = BM * kXStride, kStage = 4 * BM * 144;
    __shared__ __attribute__((aligned(16))) uint8_t lds[kBuf > kStage ? kBuf : kStage];
    uint32_t *const dpar = nullptr;  // named by the shared epilogue text for an epilogue this kernel never runs
    const uint32_t dwide = 0;

    if (blockIdx.z) batch_shift(p, blockIdx.z);
    // column blocks fastest: neighbouring workgroups share an activation tile
    const uint32_t m0 = (blockIdx.x / p.tiles_n) * BM, n0 = (blockIdx.x % p.tiles_n) * BN;
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u, wave = tid >> 6;
    const uint32_t l32 = lane & 31u, h = lane >> 5;
    const uint32_t kbytes = p.K >> 1;  // <= 128

    const __amdgpu_buffer_rsrc_t rW = make_rsrc(p.B + (uint64_t)n0 * kbytes, min(p.N - n0, (uint32_t)BN) * kbytes);
    const __amdgpu_buffer_rsrc_t rX = make_rsrc(p.A + (uint64_t)m0 * kbytes, min(p.M - m0, (uint32_t)BM) * kbytes);

    // weights: lane (l32, h) of weight tile j holds piece i = bytes [i*32 + h*16, +16) of row wave*64 + j*32 + l32
    v4u wreg[TN][4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const bool okw = i * 32 + h * 16 < kbytes;  // K % 64 == 0: a piece is all in or all out
#pragma unroll
        for (int j = 0; j < TN; ++j)
            wreg[j][i] = buf_load16(rW, okw ? (wave * 64 + j * 32 + l32) * kbytes + i * 32 + h * 16 : kOobOffset, 0);
    }
    // activations: thread (row = tid / 8 + 32 * j, piece = tid % 8) -> expanded into LDS (pieces past K as zeros)
    const uint32_t xq = tid & 7u;
    v4u xreg[NXP];
#pragma unroll
    for (int j = 0; j < NXP; ++j) {
        const uint32_t row = (tid >> 3) + j * 32;
        xreg[j] = buf_load16(rX, xq * 16 < kbytes ? row * kbytes + xq * 16 : kOobOffset, 0);
    }
#include "duq_stream_epilogue_fetch.inc"
#pragma unroll
    for (int j = 0; j < NXP; ++j) {
        const uint32_t row = (tid >> 3) + j * 32;
        v4u ev, od;
        expand_nibbles(xreg[j], ev, od);
        *reinterpret_cast<v4u *>(lds + row * kXStride + xq * 32) = ev;
        *reinterpret_cast<v4u *>(lds + row * kXStride + xq * 32 + 16) = od;
    }
    __syncthreads();

    v16i acc[TN][TM];
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int b = 0; b < TM; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[j][b][r] = 0;
    // step (i, par): weight operand = even (par 0) or odd (par 1) nibbles of piece i, activation fragment at
    // + i*64 + par*16 of the row; both sides pair the same k values
    const uint32_t fragX = l32 * kXStride + h * 32;
    auto steps = [&](int i0, int i1) {
#pragma unroll
        for (int i = i0; i < i1; ++i) {
            v4u we[TN], wo[TN];
#pragma unroll
            for (int j = 0; j < TN; ++j) expand_nibbles(wreg[j][i], we[j], wo[j]);
#pragma unroll
            for (int par = 0; par < 2; ++par) {
                v4i fx[TM];
#pragma unroll
                for (int b = 0; b < TM; ++b)
                    fx[b] = *reinterpret_cast<const v4i *>(lds + fragX + b * 32 * kXStride + i * 64 + par * 16);
#pragma unroll
                for (int b = 0; b < TM; ++b)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        acc[j][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(v4i, par ? wo[j] : we[j]), fx[b],
                                                                          acc[j][b], 0, 0, 0);
            }
        }
    };
    steps(0, 2);                   // K >= 64 always: pieces 0 and 1 (one of them zeros when K = 64)
    if (kbytes > 64) steps(2, 4);  // rows of 192 or 256 elements
    // (the activation buffer becomes the staging area of the epilogue, which waits for every wavefront first)
    constexpr bool kWideStore = true;
#include "duq_stream_epilogue_store.inc"
}

// ---------------------------------------------------------------------------------
// skinny kernel (5 <= M <= 16 on wide problems: 512 or more 16-column tiles, K <= 8192)
// ---------------------------------------------------------------------------------
// Workgroup = WAVES wavefronts that split K; it walks `tiles_per_wg` consecutive 16-column
// tiles.  Wavefront w owns 64-byte row segments [w*S, (w+1)*S), S <= 8: lane (l16, g) holds
// bytes [g*16, +16) of each.  The activation fragments of that k range do not depend on the
// column tile, so they are loaded and expanded ONCE per workgroup and stay in registers;
// per tile only the weights stream in (the next tile's loads are issued before the current
// tile's MFMAs), two MFMAs per 16-byte weight piece (even k, odd k).  Partial sums of the
// wavefronts meet in LDS (double buffered: one barrier per tile).
// Weight loads fetch whole cache lines: an instruction covers 8 rows x 128 contiguous bytes instead of the
// MFMA layout's 16 rows x 64 (half a line each); the wavefront turns the tile into the MFMA's lane layout
// through its own 8 KB of LDS (one 128-bit write and one 128-bit read per load; no barrier: the piece is
// private to the wavefront and a wavefront's LDS operations execute in order).  Slot s of a row's line holds
// its 16-byte piece s ^ ((row / 2) % 8), which makes the 16 rows x 16 bytes of a fragment read cover every bank
// once.  Measured 4-9 % faster than MFMA-layout loads from 512 column tiles on; smaller problems run the
// decode kernels (duq_decode.hip), where the extra LDS hop is not hidden.
constexpr int kSkinnySegs = 8;  // 64-byte segments per wavefront = 128-bit weight loads in flight per lane


template <int WAVES, int EPI, bool BIAS>
__global__ __launch_bounds__(WAVES * 64) void gemm_s4_skinny_kernel(DUQ_HEAD_DECL, GemmParams tail)
{
    GemmParams p = with_head(tail, DUQ_HEAD_USE);
    to_global(p.A);
    to_global(p.B);
    to_global(p.C);
    to_global(p.y);
    __shared__ v4i part[2][WAVES][64];
    __shared__ __attribute__((aligned(16))) uint8_t turn[WAVES * 8192];
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u, wave = tid >> 6;
    const uint32_t l16 = lane & 15u, g = lane >> 4;
    const uint32_t r8 = lane >> 3, j8 = lane & 7u;
    const uint32_t kbytes = p.K >> 1;
    const uint32_t segs = (kbytes + 63) / 64;
    const uint32_t seg0 = wave * kSkinnySegs;  // the launcher guarantees WAVES * kSkinnySegs >= segs
    const uint32_t tiles_per_wg = p.tiles_m;   // (field reused: column tiles per workgroup)
    const uint32_t ntiles = (p.N + 15) / 16;
    const uint32_t tile0 = blockIdx.x * tiles_per_wg;
    const uint32_t tile_end = min(tile0 + tiles_per_wg, ntiles);

    // 32-bit byte offsets over the whole tensors: the dispatcher only comes here while N * K / 2 < 2^32 - 256
    const __amdgpu_buffer_rsrc_t rW = make_rsrc(p.B, p.N * kbytes);  // rows past N read as zero
    const __amdgpu_buffer_rsrc_t rX = make_rsrc(p.A, p.M * kbytes);  // rows past M read as zero

    // activations of this wavefront's k range: once per workgroup
    v4u xe[kSkinnySegs], xo[kSkinnySegs];
#pragma unroll
    for (int u = 0; u < kSkinnySegs; ++u) {
        const uint32_t off = (seg0 + u) * 64 + g * 16;
        const bool ok = seg0 + u < segs && off < kbytes;
        const v4u x = buf_load16(rX, ok ? l16 * kbytes + off : kOobOffset, 0);
        expand_nibbles(x, xe[u], xo[u]);
    }

    auto load_tile = [&](uint32_t tile, v4u(&w)[kSkinnySegs]) {
        // load u = 2 * line + half: rows 8 * half + r8 of the tile, slot j8 of line `line` of this wavefront's range
#pragma unroll
        for (int u = 0; u < kSkinnySegs; ++u) {
            const uint32_t rt = (u & 1) * 8 + r8, row = tile * 16 + rt;
            const uint32_t off = seg0 * 64 + (u >> 1) * 128 + ((j8 ^ ((rt >> 1) & 7u)) << 4);
            const bool ok = tile < tile_end && row < p.N && off < kbytes;
            w[u] = buf_load16_aux<DUQ_SKINNY_WLOAD_AUX>(rW, ok ? row * kbytes + off : kOobOffset, 0);
        }
    };
    auto compute_tile = [&](uint32_t tile, const v4u(&w)[kSkinnySegs], uint32_t buf) {
        v4i acc = v4i{0, 0, 0, 0};
        uint8_t *mine = turn + wave * 8192;
#pragma unroll
        for (int u = 0; u < kSkinnySegs; ++u) *reinterpret_cast<v4u *>(mine + u * 1024 + lane * 16) = w[u];
#pragma unroll
        for (int u = 0; u < kSkinnySegs; ++u) {
            // segment u = 64 bytes: half (u % 2) of line u / 2; this lane's row l16 sits in load 2 * line + l16 / 8
            const uint32_t piece = (u & 1) * 4 + g;
            const v4u raw = *reinterpret_cast<const v4u *>(mine + ((u >> 1) * 2 + (l16 >> 3)) * 1024 + (l16 & 7u) * 128 +
                                                           ((piece ^ ((l16 >> 1) & 7u)) << 4));
            v4u we, wo;
            expand_nibbles(raw, we, wo);
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(v4i, we), __builtin_bit_cast(v4i, xe[u]), acc,
                                                        0, 0, 0);
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(v4i, wo), __builtin_bit_cast(v4i, xo[u]), acc,
                                                        0, 0, 0);
        }
        // every wavefront parks its 16 x 16 partial tile, then the first 256 threads each
        // finish one output element (sum over wavefronts, epilogue, store): no wavefront
        // is a serial bottleneck
        part[buf][wave][lane] = acc;
        __syncthreads();
        if (tid < 256) {
            const uint32_t src_lane = tid >> 2, r = tid & 3u;
            int sum = 0;
#pragma unroll
            for (int w2 = 0; w2 < WAVES; ++w2) sum += part[buf][w2][src_lane][r];
            sum >>= 8;
            const uint32_t m = src_lane & 15u, n = tile * 16 + (src_lane >> 4) * 4 + r;
            if (m < p.M && n < p.N) {
                if (EPI < 0) {
                    p.C[(uint64_t)m * p.N + n] = sum;
                } else {
                    constexpr int MODE = EPI < 0 ? 0 : EPI;
                    const ColParams c = load_col<MODE, BIAS>(p.epi.s_col_1, p.epi.z_col_1, p.epi.s_col_2,
                                                             p.epi.z_col_2, p.epi.bias, n, p.epi.rs_col);
                    p.y[(uint64_t)m * p.N + n] = dequant_one<MODE, BIAS>(sum, load_row<MODE>(p.epi, m), c);
                }
            }
        }
    };

    // two register sets alternate so that one tile's loads are in flight during the other's MFMAs
    v4u w0[kSkinnySegs], w1[kSkinnySegs];
    load_tile(tile0, w0);
    for (uint32_t t = tile0; t < tile_end; t += 2) {
        load_tile(t + 1, w1);
        compute_tile(t, w0, 0);
        load_tile(t + 2, w0);
        if (t + 1 < tile_end) compute_tile(t + 1, w1, 1);
    }
}

// ---------------------------------------------------------------------------------
// ring kernel (17 <= M <= 256 on narrow problems, and M <= 16 with rows of 12289..16384 elements)
// ---------------------------------------------------------------------------------
// The packed activations of all 16*RB rows sit in LDS for the whole K range (rows padded so that
// 16 rows x 16 bytes cover every bank once); a wavefront owns a 16-column tile and a K slice
// and streams the weights of that slice through a ring of kRing 128-bit loads per lane that is
// refilled slot by slot, across tile boundaries too, so the loads in flight never drain.  Every
// weight fragment is expanded once and multiplied with the RB activation fragments read from
// LDS (one expansion each).  No barrier inside the K loop; when several wavefronts split K for
// a tile their partial sums meet in LDS once per tile.  More rows than 16*RB are covered by
// blockIdx.y (groups of 16*RB rows, each streaming the weights again).
constexpr int kRing = 8;  // 128-bit weight loads in flight per lane

template <int XBYTES, int RB, int EPI, bool BIAS>
__global__ __launch_bounds__(256) void gemm_s4_ring_kernel(DUQ_HEAD_DECL, GemmParams tail)
{
    GemmParams p = with_head(tail, DUQ_HEAD_USE);
    to_global(p.A);
    to_global(p.B);
    to_global(p.C);
    to_global(p.y);
    constexpr uint32_t WAVES = 4, T = WAVES * 64;
    constexpr uint32_t XS = XBYTES + 16;  // LDS row stride = 16 (mod 256)
    __shared__ __attribute__((aligned(16))) uint8_t xs[16 * RB * XS];
    __shared__ v4i part[WAVES][RB][64];
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u, wave = tid >> 6;
    const uint32_t l16 = lane & 15u, g = lane >> 4;
    const uint32_t kbytes = p.K >> 1;
    const uint32_t segs = (kbytes + 63) / 64;
    const uint32_t kslices = p.tiles_m;  // (fields reused) wavefronts that split K for one tile: 1, 2 or 4
    const uint32_t items = p.tiles_n;    // tiles each wavefront walks through
    const uint32_t tiles_per_wg = WAVES / kslices;
    const uint32_t slice = wave % kslices, tsub = wave / kslices;
    const uint32_t sps = (segs + kslices - 1) / kslices;  // 64-byte segments per slice
    const uint32_t seg_lo = slice * sps;
    const uint32_t nblk = (sps + kRing - 1) / kRing;
    const uint32_t m_base = blockIdx.y * (16 * RB);

    const __amdgpu_buffer_rsrc_t rW = make_rsrc(p.B, p.N * kbytes);  // rows past N read as zero
    const __amdgpu_buffer_rsrc_t rX = make_rsrc(p.A, p.M * kbytes);  // rows past M read as zero

    v4u ring[kRing];
    auto tile_of = [&](uint32_t it) { return (blockIdx.x * items + it) * tiles_per_wg + tsub; };
    auto issue = [&](uint32_t it, uint32_t blk, int j) {
        const uint32_t row = tile_of(it) * 16 + l16;
        const uint32_t sg = blk * kRing + j;
        const uint32_t off = (seg_lo + sg) * 64 + g * 16;
        const bool ok = it < items && row < p.N && sg < sps && off < kbytes;
        ring[j] = buf_load16_aux<DUQ_RING_WLOAD_AUX>(rW, ok ? row * kbytes + off : kOobOffset, 0);
    };
#pragma unroll
    for (int j = 0; j < kRing; ++j) issue(0, 0, j);  // the first weights are under way before the activations

    {
        const uint32_t ppr = kbytes >> 4;  // 16-byte pieces per row
        for (uint32_t c = tid; c < ppr; c += T) {
#pragma unroll
            for (int r0 = 0; r0 < 16 * RB; r0 += 16) {
                v4u v[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) v[r] = buf_load16(rX, (m_base + r0 + r) * kbytes + c * 16, 0);
#pragma unroll
                for (int r = 0; r < 16; ++r) *reinterpret_cast<v4u *>(xs + (r0 + r) * XS + c * 16) = v[r];
            }
        }
    }
    __syncthreads();

    const bool vec_ok = (EPI < 0) ? (p.N % 4 == 0 && reinterpret_cast<uintptr_t>(p.C) % 16 == 0)
                                  : (p.N % 4 == 0 && reinterpret_cast<uintptr_t>(p.y) % 8 == 0);
    const uint32_t xbase = l16 * XS + g * 16;
    for (uint32_t it = 0; it < items; ++it) {
        v4i acc[RB];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) acc[rb] = v4i{0, 0, 0, 0};
        for (uint32_t blk = 0; blk < nblk; ++blk) {
            const bool last = blk + 1 == nblk;
            const uint32_t nit = last ? it + 1 : it, nb = last ? 0 : blk + 1;
#pragma unroll
            for (int j = 0; j < kRing; ++j) {
                const v4u w = ring[j];
                issue(nit, nb, j);
                // segments past the slice carry zero weights; their activation read only has to stay inside the row
                const uint32_t xoff = min((seg_lo + blk * kRing + j) * 64, (uint32_t)XBYTES - 64);
                v4u we, wo;
                expand_nibbles(w, we, wo);
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) {
                    const v4u x = *reinterpret_cast<const v4u *>(xs + rb * 16 * XS + xbase + xoff);
                    v4u xe, xo;
                    expand_nibbles(x, xe, xo);
                    acc[rb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(v4i, we),
                                                                   __builtin_bit_cast(v4i, xe), acc[rb], 0, 0, 0);
                    acc[rb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(v4i, wo),
                                                                   __builtin_bit_cast(v4i, xo), acc[rb], 0, 0, 0);
                }
            }
        }
        const uint32_t tile = tile_of(it);
        if (kslices > 1) {
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) part[wave][rb][lane] = acc[rb];
            __syncthreads();
            if (slice == 0)
                for (uint32_t s2 = 1; s2 < kslices; ++s2)
#pragma unroll
                    for (int rb = 0; rb < RB; ++rb) {
                        const v4i o = part[wave + s2][rb][lane];
#pragma unroll
                        for (int r = 0; r < 4; ++r) acc[rb][r] += o[r];
                    }
            __syncthreads();  // the partial sums are consumed before the next tile overwrites them
        }
        if (slice == 0) {
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[rb][r] >>= 8;
                store_quad<EPI, BIAS>(p, m_base + rb * 16 + l16, tile * 16 + g * 4, acc[rb], vec_ok);
            }
        }
    }
}

// ---------------------------------------------------------------------------------
// dot kernel (M <= 4, rows longer than 16384 elements): weight streaming on v_dot8_i32_i4
// ---------------------------------------------------------------------------------
// The signed 4-bit dot product instruction consumes packed nibbles as they lie in memory,
// so nothing is expanded and no MFMA is needed: the kernel is a pure HBM stream.
// Workgroup = 4 wavefronts = 8 weight rows, K split four ways.  Lane (r8, j) walks its
// quarter of row r8 in 128-byte steps, loading bytes [step*128 + j*16, +16): one wavefront
// load is eight full cache lines.  Eight loads per lane are kept in flight (a register
// ring), and with ~40 VGPRs eight wavefronts fit on a SIMD, so a CU keeps > 100 KB of
// weights in flight.  The M activation rows sit in LDS (lanes of different rows read the
// same address: a broadcast).  Partial sums meet through three lane shuffles and one LDS hop.
constexpr int kDotRing = 8;

template <int MROWS, int EPI, bool BIAS>
__global__ __launch_bounds__(256) void gemv_s4_dot_kernel(DUQ_HEAD_DECL, GemmParams tail)
{
    GemmParams p = with_head(tail, DUQ_HEAD_USE);
    to_global(p.A);
    to_global(p.B);
    to_global(p.C);
    to_global(p.y);
    extern __shared__ __attribute__((aligned(16))) uint8_t xs[];  // [MROWS][xstride] packed activations
    __shared__ int part[4][8][MROWS];
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u, wave = tid >> 6;
    const uint32_t r8 = lane >> 3, j = lane & 7u;
    const uint32_t kbytes = p.K >> 1;
    const uint32_t nsteps_all = (kbytes + 127) / 128;
    const uint32_t xstride = nsteps_all * 128;
    const uint32_t per = (nsteps_all + 3) / 4;
    const uint32_t step0 = wave * per;
    const uint32_t nsteps = step0 < nsteps_all ? min(per, nsteps_all - step0) : 0;
    const uint32_t n = blockIdx.x * 8 + r8;

    const __amdgpu_buffer_rsrc_t rW = make_rsrc(p.B, p.N * kbytes);  // rows past N read as zero
    const uint32_t wbase = n * kbytes + j * 16;

    auto w_off = [&](uint32_t s) -> uint32_t {  // step s of this wavefront's slice
        const uint32_t off = (step0 + s) * 128 + j * 16;
        return (s < nsteps && off < kbytes && n < p.N) ? wbase + (step0 + s) * 128 : kOobOffset;
    };

    v4u ring[kDotRing];
#pragma unroll
    for (int u = 0; u < kDotRing; ++u) ring[u] = buf_load16_aux<DUQ_DOT_WLOAD_AUX>(rW, w_off(u), 0);

    // activations -> LDS (all rows, whole K), zero beyond the row end
    for (uint32_t i = tid; i < MROWS * (xstride / 16); i += 256) {
        const uint32_t m = i / (xstride / 16), o = (i % (xstride / 16)) * 16;
        v4u v = v4u{0u, 0u, 0u, 0u};
        if (m < p.M && o < kbytes) v = *reinterpret_cast<const v4u *>(p.A + (uint64_t)m * kbytes + o);
        *reinterpret_cast<v4u *>(xs + m * xstride + o) = v;
    }
    __syncthreads();

    int acc[MROWS];
#pragma unroll
    for (int m = 0; m < MROWS; ++m) acc[m] = 0;

    for (uint32_t s = 0; s < nsteps; s += kDotRing) {
#pragma unroll
        for (int u = 0; u < kDotRing; ++u) {
            const v4u w = ring[u];
            ring[u] = buf_load16_aux<DUQ_DOT_WLOAD_AUX>(rW, w_off(s + u + kDotRing), 0);
            const uint32_t xo = (step0 + s + u) * 128 + j * 16;
            if (s + u < nsteps) {
#pragma unroll
                for (int m = 0; m < MROWS; ++m) {
                    const v4u x = *reinterpret_cast<const v4u *>(xs + m * xstride + xo);
#pragma unroll
                    for (int d = 0; d < 4; ++d) acc[m] = __builtin_amdgcn_sdot8((int)w[d], (int)x[d], acc[m], false);
                }
            }
        }
    }

    // the 8 lanes of a row, then the 4 wavefronts
#pragma unroll
    for (int m = 0; m < MROWS; ++m) {
        acc[m] += __shfl_xor(acc[m], 1, kWave);
        acc[m] += __shfl_xor(acc[m], 2, kWave);
        acc[m] += __shfl_xor(acc[m], 4, kWave);
    }
    if (j == 0) {
#pragma unroll
        for (int m = 0; m < MROWS; ++m) part[wave][r8][m] = acc[m];
    }
    __syncthreads();
    if (tid < 8 * MROWS) {
        const uint32_t rr = tid / MROWS, m = tid % MROWS;
        const uint32_t nn = blockIdx.x * 8 + rr;
        if (nn < p.N && m < p.M) {
            const int v = part[0][rr][m] + part[1][rr][m] + part[2][rr][m] + part[3][rr][m];
            if (EPI < 0) {
                p.C[(uint64_t)m * p.N + nn] = v;
            } else {
                constexpr int MODE = EPI < 0 ? 0 : EPI;
                const ColParams c = load_col<MODE, BIAS>(p.epi.s_col_1, p.epi.z_col_1, p.epi.s_col_2, p.epi.z_col_2,
                                                         p.epi.bias, nn, p.epi.rs_col);
                p.y[(uint64_t)m * p.N + nn] = dequant_one<MODE, BIAS>(v, load_row<MODE>(p.epi, m), c);
            }
        }
    }
}

// ---------------------------------------------------------------------------------
// dispatch
// ---------------------------------------------------------------------------------
// Which kernel family takes a shape.  Host arithmetic only, so that the rule can be tested without a GPU:
// every kernel whose weight offsets are 32-bit (decode, dot, ring: row * K/2 + offset, and a buffer descriptor
// over the whole tensor) is reachable only while the packed weights stay below 4 GiB - 256 (the out-of-range
// marker); larger tensors go to the stream / tile kernels, whose descriptors and pointers are per tile
// (64-bit base, 32-bit offsets inside 256 rows).
int select_gemm_kernel(uint32_t M, uint32_t N, uint32_t K)
{
    const uint64_t wbytes = (uint64_t)N * (K / 2);
    const bool small_offsets = wbytes < 0xFFFFFF00ull && K > 0;
    // decode.  Rows kernel for up to four rows (8 KB of every weight row per wavefront); above, the MFMA decode
    // kernel (6 KB per row over eight wavefronts), with two to four row tiles against the same weight fragments
    // for 17..64 rows as far as the fragments fit in registers (64 rows of at most 8192 elements, 48 of at most
    // 12288).  Two exceptions, both measured: 9..16 rows on very wide layers run the skinny kernel (whole-line
    // weight loads, 5 % faster at N = 28672, K = 4096), and the long-row forms (more than 32 rows of more than 4096
    // elements, any of more than 8192) need 192 column tiles: on narrower layers the ring kernel, which splits K
    // over workgroups, is ahead (48 x 1024 x 8192: 7.9 against 10.2 us; 48 x 3072 x 12288: 20.6 against 14.1).
    if (M <= 4 && K <= 16384 && small_offsets) return kKernelDecodeRows;
    if (M <= 16 && small_offsets) {
        if (M > 8 && (N + 15) / 16 >= 1536 && K <= 4096) return kKernelSkinny;
        if (K <= 12288) return kKernelDecodeMfma;
    }
    if (M <= 64 && small_offsets) {
        if (K <= 4096 || (K <= 8192 && M <= 32)) return kKernelDecodeMfma;
        if ((N + 15) / 16 >= 192 && (K <= 8192 || (K <= 12288 && M <= 48))) return kKernelDecodeMfma;
    }
    const uint32_t xstride = ((K / 2 + 127) / 128) * 128;
    // dot kernel: up to four rows too long for the decode kernels
    if (M <= 4 && small_offsets && 4 * xstride <= 60 * 1024) return kKernelDot;
    // more than 64 rows whose 64 x 128 tiles make one round of 64..256 workgroups: the stream kernel on those tiles
    // (measured against the ring kernel, N = 4096: 128 x 4096 11.9 against 14.6 us, 192 x 4096 12.1 against 18.3,
    // 128 x 11008 (K) 25.1 against 42.2; with fewer tiles the ring kernel, which splits K over workgroups, is far
    // ahead: 200 x 520 x 8192 8.2 against 28.8 us)
    const uint32_t narrow_tiles = ((M + 63) / 64) * ((N + 127) / 128);
    const bool narrow_round = M > 64 && narrow_tiles >= 64 && narrow_tiles <= 256;
    {
        // ring kernel: 17..256 rows in groups whose packed activations fit in LDS (a few groups only, or a
        // problem too narrow to fill the chip with stream-kernel tiles)
        const uint32_t rb_all = (M + 15) / 16;
        const uint32_t rb_max = K <= 4096 ? 4 : (K <= 8192 ? 2 : 1);  // 16-row blocks whose activations fit in LDS
        const uint32_t rb = std::min(rb_all, rb_max);
        const uint32_t row_groups = (rb_all + rb - 1) / rb;
        // (several row groups re-stream the weights: with enough column tiles to fill the chip the stream
        // kernel's 32-row tiles are cheaper then)
        const uint32_t tiles32 = ((M + 31) / 32) * ((N + 255) / 256);
        const bool few_groups = row_groups <= 2 || (row_groups <= 6 && tiles32 < 64) || tiles32 < 48;
        const bool mid_rows = M > 16 && M <= 256 && few_groups && !(row_groups > 1 && tiles32 >= 128);
        const bool long_rows = M <= 16 && K > 8192;  // 5..16 rows of 12289..16384 elements
        if ((long_rows || mid_rows) && K <= 16384 && small_offsets && !narrow_round) return kKernelRing;
    }
    auto tiles = [&](uint32_t bm, uint32_t bn) { return ((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
    if (narrow_round || (M > 32 && tiles(32, 256) >= 32)) return kKernelStream;
    return kKernelTile;
}

// batch > 1: `batch` problems of one shape, tensors contiguous over the batch, one launch (blockIdx.z is the
// problem): stream or tile kernel only, the choice made on the tiles of the whole batch.
template <int EPI, bool BIAS>
static void launch_epi(GemmParams &p, hipStream_t stream, uint32_t batch = 1)
{
    const int kernel = batch > 1 ? (p.M > 32 && ((p.M + 31) / 32) * ((p.N + 255) / 256) * batch >= 32 ? kKernelStream : kKernelTile)
                                 : select_gemm_kernel(p.M, p.N, p.K);
    // (EPI 5, the dual-uniform row-sum epilogue, exists in the stream kernel only: gemm_fuses_dual_rowsum)
    if constexpr (EPI != 5) {
    if (kernel == kKernelDot) {
        const uint32_t xstride = ((p.K / 2 + 127) / 128) * 128;
        const dim3 grid((p.N + 7) / 8);
        if (p.M == 1)
            DUQ_LAUNCH_HEAD((gemv_s4_dot_kernel<1, EPI, BIAS>), grid, dim3(256), 1 * xstride, stream, p);
        else if (p.M == 2)
            DUQ_LAUNCH_HEAD((gemv_s4_dot_kernel<2, EPI, BIAS>), grid, dim3(256), 2 * xstride, stream, p);
        else
            DUQ_LAUNCH_HEAD((gemv_s4_dot_kernel<4, EPI, BIAS>), grid, dim3(256), 4 * xstride, stream, p);
        return;
    }
    if (kernel == kKernelSkinny) {
        const uint32_t ntiles = (p.N + 15) / 16;
        const uint32_t segs = (p.K / 2 + 63) / 64;
        // several column tiles per workgroup (activations are fetched and expanded once per workgroup); at least
        // ~2 workgroups per CU stay.  Long rows (8 wavefronts per workgroup, one workgroup per CU): whole rounds
        // of 256 workgroups, at most 8 tiles each.
        uint32_t tpw = ntiles >= 6144 ? 8 : (ntiles >= 1536 ? 4 : (ntiles >= 640 ? 2 : 1));
        if (segs > 4 * kSkinnySegs) {
            const uint32_t rounds = (ntiles + 2047) / 2048;
            tpw = (ntiles + 256 * rounds - 1) / (256 * rounds);
        }
        p.tiles_m = tpw;
        const dim3 grid((ntiles + tpw - 1) / tpw);
        if (segs <= 4 * kSkinnySegs)
            DUQ_LAUNCH_HEAD((gemm_s4_skinny_kernel<4, EPI, BIAS>), grid, dim3(256), 0, stream, p);
        else
            DUQ_LAUNCH_HEAD((gemm_s4_skinny_kernel<8, EPI, BIAS>), grid, dim3(512), 0, stream, p);
        return;
    }
    if (kernel == kKernelRing) {
        const uint32_t rb_all = (p.M + 15) / 16;
        const uint32_t rb_max = p.K <= 4096 ? 4 : (p.K <= 8192 ? 2 : 1);
        const uint32_t rb = std::min(rb_all, rb_max);
        const uint32_t row_groups = (rb_all + rb - 1) / rb;
        const uint32_t ntiles = (p.N + 15) / 16;
        const uint32_t segs = (p.K / 2 + 63) / 64;
        // wavefronts splitting K for one tile: as few as give the chip ~2048 wavefronts, slices of at
        // least 512 bytes per row
        uint32_t kslices = 1;
        while (ntiles * kslices < 2048 && kslices < 4 && segs / (kslices * 2) >= (uint32_t)kRing) kslices *= 2;
        const uint32_t groups = (ntiles + 4 / kslices - 1) / (4 / kslices);
        const uint32_t xbytes = p.K <= 4096 ? 2048 : (p.K <= 8192 ? 4096 : 8192);
        const uint32_t lds = 16 * rb * (xbytes + 16) + 4 * rb * 1024;
        const uint32_t slots = 256 * std::max(1u, std::min(8u, (160u * 1024) / lds));
        p.tiles_m = kslices;
        p.tiles_n = (groups + slots - 1) / slots;
        const dim3 grid((groups + p.tiles_n - 1) / p.tiles_n, row_groups);
#define DUQ_RING(X, R) DUQ_LAUNCH_HEAD((gemm_s4_ring_kernel<X, R, EPI, BIAS>), grid, dim3(256), 0, stream, p)
        if (xbytes == 8192) DUQ_RING(8192, 1);
        else if (xbytes == 4096) DUQ_RING(4096, 2);
        else if (rb == 2) DUQ_RING(2048, 2);
        else if (rb == 3) DUQ_RING(2048, 3);
        else DUQ_RING(2048, 4);
#undef DUQ_RING
        return;
    }
    }
    // Stream kernel: the tile that select_stream_tile prices cheapest; small problems (few column tiles) stay on
    // the tile kernels.
    auto tiles = [&](uint32_t bm, uint32_t bn) { return ((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn) * batch; };
    int best_tm = 0;
    bool half_width = false;  // 128-column tiles
    if (kernel == kKernelStream) {
        const StreamTile tile = select_stream_tile(p.M, p.N, p.K, batch, EPI == 5);
        if constexpr (EPI != 5) {
            if (tile.rows == 256) {
                p.tiles_m = (p.M + 255) / 256;
                p.tiles_n = (p.N + 255) / 256;
                DUQ_LAUNCH_HEAD((gemm_s4_stream256_kernel<EPI, BIAS>), dim3(p.tiles_m * p.tiles_n, 1, batch), dim3(256), 0,
                                stream, p);
                return;
            }
        }
        best_tm = (int)(tile.rows / 32);
        half_width = tile.cols == 128;
    }
    if constexpr (EPI != 5) if (best_tm && p.K <= 256) {
        // rows of at most 256 elements: one chunk, the launch is its output stores: the short-row kernel with 64-row
        // tiles (measured on 32 products of 2048 x 2048 x 128: 86 us against 95 us on the stream kernel's 64-row tiles)
        p.tiles_m = (p.M + 63) / 64;
        p.tiles_n = (p.N + 255) / 256;
        DUQ_LAUNCH_HEAD((gemm_s4_shortk_kernel<2, EPI, BIAS>), dim3(p.tiles_m * p.tiles_n, 1, batch), dim3(256), 0,
                           stream, p);
        return;
    }
    if (best_tm && half_width) {
        p.tiles_m = (p.M + 32 * best_tm - 1) / (32 * best_tm);
        p.tiles_n = (p.N + 127) / 128;
        const dim3 grid(p.tiles_m * p.tiles_n, 1, batch);
        if (best_tm == 4)
            DUQ_LAUNCH_HEAD((gemm_s4_stream_kernel<4, EPI, BIAS, 1>), grid, dim3(256), 0, stream, p);
        else
            DUQ_LAUNCH_HEAD((gemm_s4_stream_kernel<2, EPI, BIAS, 1>), grid, dim3(256), 0, stream, p);
    } else if (best_tm) {
        p.tiles_m = (p.M + 32 * best_tm - 1) / (32 * best_tm);
        p.tiles_n = (p.N + 255) / 256;
        const dim3 grid(p.tiles_m * p.tiles_n, 1, batch);
        if (best_tm == 4)
            DUQ_LAUNCH_HEAD((gemm_s4_stream_kernel<4, EPI, BIAS>), grid, dim3(256), 0, stream, p);
        else if (best_tm == 2)
            DUQ_LAUNCH_HEAD((gemm_s4_stream_kernel<2, EPI, BIAS>), grid, dim3(256), 0, stream, p);
        else
            DUQ_LAUNCH_HEAD((gemm_s4_stream_kernel<1, EPI, BIAS>), grid, dim3(256), 0, stream, p);
    } else if constexpr (EPI != 5) {
        if (tiles(128, 256) >= 256 && p.M > 64) {
            p.tiles_m = (p.M + 127) / 128;
            p.tiles_n = (p.N + 255) / 256;
            DUQ_LAUNCH_HEAD((gemm_s4_tile_kernel<128, 256, EPI, BIAS>), dim3(p.tiles_m * p.tiles_n, 1, batch), dim3(256),
                               0, stream, p);
        } else if (tiles(128, 128) >= 256 && p.M > 64) {
            p.tiles_m = (p.M + 127) / 128;
            p.tiles_n = (p.N + 127) / 128;
            DUQ_LAUNCH_HEAD((gemm_s4_tile_kernel<128, 128, EPI, BIAS>), dim3(p.tiles_m * p.tiles_n, 1, batch), dim3(256),
                               0, stream, p);
        } else {
            p.tiles_m = (p.M + 63) / 64;
            p.tiles_n = (p.N + 63) / 64;
            DUQ_LAUNCH_HEAD((gemm_s4_tile_kernel<64, 64, EPI, BIAS>), dim3(p.tiles_m * p.tiles_n, 1, batch), dim3(256), 0,
                               stream, p);
        }
    }
}

int launch_gemm_s4(const uint8_t *A, const uint8_t *B, uint32_t M, uint32_t N, uint32_t K, int32_t *out_acc,
                   const Epilogue *epi, uint16_t *y, hipStream_t stream)
{
    return launch_gemm_s4_batched(A, B, M, N, K, 1, out_acc, epi, y, stream);
}

int launch_gemm_s4_batched(const uint8_t *A, const uint8_t *B, uint32_t M, uint32_t N, uint32_t K, uint32_t batch,
                           int32_t *out_acc, const Epilogue *epi, uint16_t *y, hipStream_t stream)
{
    if (M == 0 || N == 0 || batch == 0) return 0;
    if (batch == 1) {
        const int kernel = select_gemm_kernel(M, N, K);
        if (kernel == kKernelDecodeRows || kernel == kKernelDecodeMfma)
            return launch_decode_s4(A, B, M, N, K, out_acc, epi, y, stream);
    }
    GemmParams p{};
    p.A = A;
    p.B = B;
    p.M = M;
    p.N = N;
    p.K = K;
    p.C = out_acc;
    p.y = y;
    if (epi) p.epi = *epi;
    if (out_acc) {
        launch_epi<-1, false>(p, stream, batch);
    } else {
        const bool bias = epi->bias != nullptr;
#define DUQ_GEMM(MODE)                             \
    case MODE:                                     \
        if (bias)                                  \
            launch_epi<MODE, true>(p, stream, batch);  \
        else                                       \
            launch_epi<MODE, false>(p, stream, batch); \
        break;
        switch (epi->mode) {
            DUQ_GEMM(0)
            DUQ_GEMM(1)
            DUQ_GEMM(2)
            DUQ_GEMM(3)
            DUQ_GEMM(4)
        case 5:
            if (batch != 1 || !gemm_fuses_dual_rowsum(M, N, K)) return (int)hipErrorInvalidValue;
            if (bias)
                launch_epi<5, true>(p, stream, 1);
            else
                launch_epi<5, false>(p, stream, 1);
            break;
        default:
            return (int)hipErrorInvalidValue;
        }
#undef DUQ_GEMM
    }
    return (int)hipGetLastError();
}

}  // namespace duq
