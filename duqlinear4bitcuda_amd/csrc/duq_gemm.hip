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
// Two kernels:
//  * tile kernel (prefill, M > 16): BM x BN x 128 tiles, 4 wavefronts (2 x 2), packed
//    nibbles are expanded to bytes on the way from global memory into LDS, LDS rows are
//    padded to 144 B so that the 128-bit fragment reads are bank-conflict free, LDS is
//    double buffered and the next tile's global loads are in flight during the MFMAs.
//    The weight operand goes to the MFMA "A" side, so each lane ends up with four
//    consecutive output columns of one row and stores them as one vector.
//  * skinny kernel (decode, M <= 16): HBM-bound weight streaming.  One workgroup owns 16
//    output columns, its wavefronts split K, every lane issues all of its 128-bit weight
//    loads before the first MFMA, fragments go from global memory straight to registers
//    (no LDS for operands), partial sums meet in LDS once at the end.
#include "duq_epilogue.h"
#include "duq_launch.h"
#include <cstdlib>
#include <type_traits>

namespace duq {

constexpr uint32_t kNibbleMask = 0xF0F0F0F0u;

struct GemmParams {
    const uint8_t *A;  // activations [M, K/2]
    const uint8_t *B;  // weights     [N, K/2]
    uint32_t M, N, K;
    int32_t *C;        // int32 out (EPI < 0)
    uint16_t *y;       // fp16 out  (EPI >= 0)
    Epilogue epi;
    uint32_t tiles_m, tiles_n;
};

__device__ __forceinline__ void expand_nibbles(const v4u w, v4u &even, v4u &odd)
{
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        even[i] = (w[i] << 4) & kNibbleMask;
        odd[i] = w[i] & kNibbleMask;
    }
}

// Workgroup id -> tile id.  Consecutive workgroup ids land on consecutive XCDs (8 of them,
// each with its own L2), so ids are regrouped to give every XCD one contiguous range of
// tiles; tiles inside a range walk down a band of 8 tile-rows first, which keeps the A and
// B panels an XCD touches compact.
__device__ __forceinline__ void tile_of_block(uint32_t bid, uint32_t tiles_m, uint32_t tiles_n, uint32_t &tm,
                                              uint32_t &tn)
{
    const uint32_t ntiles = tiles_m * tiles_n;
    const uint32_t per = ntiles / 8, rem = ntiles % 8;
    const uint32_t xcd = bid % 8, local = bid / 8;
    const uint32_t logical = xcd < rem ? xcd * (per + 1) + local : rem * (per + 1) + (xcd - rem) * per + local;
    constexpr uint32_t GM = 8;
    const uint32_t per_band = GM * tiles_n;
    const uint32_t band = logical / per_band;
    const uint32_t first_m = band * GM;
    const uint32_t band_h = min(tiles_m - first_m, GM);
    const uint32_t in_band = logical % per_band;
    tm = first_m + in_band % band_h;
    tn = in_band / band_h;
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
        const f16 s_row = bits_to_f16(p.epi.s_row[m]);
        const f16 z_row = (MODE == 1 || MODE == 3) ? bits_to_f16(p.epi.z_row[m]) : (f16)0;
        uint16_t out[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const uint32_t n = min(n0 + r, p.N - 1);
            const ColParams c = load_col<MODE, BIAS>(p.epi.s_col_1, p.epi.z_col_1, p.epi.s_col_2, p.epi.z_col_2,
                                                     p.epi.bias, n);
            out[r] = dequant_one<MODE, BIAS>(acc[r], s_row, z_row, c);
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
__global__ __launch_bounds__(256) void gemm_s4_tile_kernel(GemmParams p)
{
    constexpr int WTM = BM / 2, WTN = BN / 2;  // per-wavefront tile
    constexpr int TM = WTM / 16, TN = WTN / 16;
    constexpr int NA = BM / 64, NB = BN / 64;  // 16-byte global pieces per thread
    static_assert(BM % 64 == 0 && BN % 64 == 0, "tile shape");

    __shared__ __attribute__((aligned(16))) uint8_t lds[2][(BM + BN) * kLdsStride];

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

// ---------------------------------------------------------------------------------
// stream kernel (prefill): weights global -> registers, activations through LDS
// ---------------------------------------------------------------------------------
// Workgroup = 4 wavefronts side by side along N: every wavefront owns 16*TN weight rows
// that no other wavefront of the workgroup needs, so weight fragments never go through
// LDS: lane (l16, g) loads bytes [g*32, g*32+32) of the 128-byte row segment of a 256-k
// chunk straight into registers (two 128-bit loads = one full cache line per row and
// chunk), one chunk ahead of the MFMAs that consume them.  The 16*TM activation rows are
// shared by the four wavefronts: they are expanded to bytes once on the way into LDS
// (double buffered, rows padded to 272 B) and read back as 128-bit fragments.
// LDS traffic per 256-k chunk drops to BM*256 B written + 4*BM*256 B read.
//
// All global reads are raw buffer loads on per-workgroup descriptors that cover exactly
// the rows of this tile: rows past M or N read as zero without a branch, and the chunk
// offset rides in the scalar offset.  Only a ragged last chunk (K % 256 != 0) uses
// per-piece guarded offsets.
constexpr int kCK = 256;         // k elements per chunk (128 packed bytes per row)
constexpr int kXStride = 272;    // LDS bytes per activation row: 256 expanded + 16 pad
constexpr uint32_t kOobOffset = 0xFFFFFF00u;  // beyond any descriptor: the load returns 0

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ v4u buf_load16(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff)
{
    return __builtin_bit_cast(v4u, __builtin_amdgcn_raw_buffer_load_b128(r, (int)voff, (int)soff, 0));
}

template <int TM, int TN, int EPI, bool BIAS>
__global__ __launch_bounds__(256) void gemm_s4_stream_kernel(GemmParams p)
{
    constexpr int BM = 16 * TM;
    constexpr int WN = 16 * TN;
    constexpr int BN = 4 * WN;
    constexpr int NXP = BM / 32;  // 16-byte activation pieces per thread and chunk
    static_assert(BM % 32 == 0, "BM");

    __shared__ __attribute__((aligned(16))) uint8_t lds[2][BM * kXStride];

    uint32_t tile_m, tile_n;
    tile_of_block(blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u, wave = tid >> 6;
    const uint32_t l16 = lane & 15u, g = lane >> 4;
    const uint32_t kbytes = p.K >> 1;
    const uint32_t nfull = p.K / kCK;
    const uint32_t nchunks = (p.K + kCK - 1) / kCK;

    const __amdgpu_buffer_rsrc_t rW = make_rsrc(p.B + (uint64_t)n0 * kbytes, min(p.N - n0, (uint32_t)BN) * kbytes);
    const __amdgpu_buffer_rsrc_t rX = make_rsrc(p.A + (uint64_t)m0 * kbytes, min(p.M - m0, (uint32_t)BM) * kbytes);

    uint32_t woff[TN];
#pragma unroll
    for (int a = 0; a < TN; ++a) woff[a] = (wave * WN + a * 16 + l16) * kbytes + g * 32;
    uint32_t xoff[NXP], xlds[NXP];
    const uint32_t xq = tid & 7u;  // which 16-byte piece of the 128-byte row segment
#pragma unroll
    for (int i = 0; i < NXP; ++i) {
        const uint32_t row = (tid >> 3) + i * 32;
        xoff[i] = row * kbytes + xq * 16;
        xlds[i] = row * kXStride + xq * 32;
    }

    v4u wreg[TN][2];
    v4u xreg[NXP];

    // PF selects how the NEXT chunk is fetched: 0 none, 1 full chunk (no guards), 2 ragged
    // last chunk (pieces past the row end are redirected out of bounds and read as zero).
    auto load_w = [&](auto pf, int j, uint32_t c) {
        constexpr int PF = decltype(pf)::value;
        const uint32_t koff = c * (kCK / 2);
        if (PF == 1) {
#pragma unroll
            for (int a = 0; a < TN; ++a) wreg[a][j] = buf_load16(rW, woff[a] + j * 16, koff);
        } else if (PF == 2) {
            const bool ok = koff + g * 32 + j * 16 < kbytes;  // K % 64 == 0: all in or all out
#pragma unroll
            for (int a = 0; a < TN; ++a) wreg[a][j] = buf_load16(rW, ok ? woff[a] + j * 16 : kOobOffset, koff);
        }
    };
    auto load_x = [&](auto pf, uint32_t c) {
        constexpr int PF = decltype(pf)::value;
        const uint32_t koff = c * (kCK / 2);
        if (PF == 1) {
#pragma unroll
            for (int i = 0; i < NXP; ++i) xreg[i] = buf_load16(rX, xoff[i], koff);
        } else if (PF == 2) {
            const bool okx = koff + xq * 16 < kbytes;
#pragma unroll
            for (int i = 0; i < NXP; ++i) xreg[i] = buf_load16(rX, okx ? xoff[i] : kOobOffset, koff);
        }
    };
    auto store_x = [&](uint32_t buf) {
        uint8_t *base = lds[buf];
#pragma unroll
        for (int i = 0; i < NXP; ++i) {
            v4u ev, od;
            expand_nibbles(xreg[i], ev, od);
            *reinterpret_cast<v4u *>(base + xlds[i]) = ev;
            *reinterpret_cast<v4u *>(base + xlds[i] + 16) = od;
        }
    };

    v4i acc[TN][TM];
#pragma unroll
    for (int a = 0; a < TN; ++a)
#pragma unroll
        for (int b = 0; b < TM; ++b) acc[a][b] = v4i{0, 0, 0, 0};

    const uint32_t fragX = l16 * kXStride + g * 64;  // fragment step*16 with step = j*2+par

    // One chunk = 4 MFMA steps (j, par), each TM groups of TN MFMAs.  The instruction order
    // is fixed by hand (scheduling fences around every MFMA group): while the TN MFMAs of a
    // group run, the next step's activation fragment for the same group index is read from
    // LDS, the weight registers of half j are refilled for the next chunk right after they
    // were expanded, and the next chunk's activations are expanded and written to the other
    // LDS buffer inside the last step.  MFMAs are issued through inline assembly with the
    // accumulators tied to the accumulation register file, so they never move.
    auto body = [&](auto pf, uint32_t c) {
        constexpr int PF = decltype(pf)::value;
        const uint32_t cur = c & 1u;
        const uint8_t *base = lds[cur] + fragX;
        uint8_t *nbase = lds[cur ^ 1u];
        load_x(pf, c + 1);
        v4i fx[2][TM];
#pragma unroll
        for (int b = 0; b < TM; ++b) fx[0][b] = *reinterpret_cast<const v4i *>(base + b * 16 * kXStride);
        v4u we[TN], wo[TN];
#pragma unroll
        for (int step = 0; step < 4; ++step) {
            const int j = step >> 1, par = step & 1;
            if (par == 0) {
#pragma unroll
                for (int a = 0; a < TN; ++a) expand_nibbles(wreg[a][j], we[a], wo[a]);
                load_w(pf, j, c + 1);
            }
#pragma unroll
            for (int b = 0; b < TM; ++b) {
                if (step < 3)
                    fx[(step + 1) & 1][b] =
                        *reinterpret_cast<const v4i *>(base + b * 16 * kXStride + (step + 1) * 16);
                if (PF != 0 && step == 3 && b < NXP) {  // next chunk's activations -> LDS
                    v4u ev, od;
                    expand_nibbles(xreg[b], ev, od);
                    *reinterpret_cast<v4u *>(nbase + xlds[b]) = ev;
                    *reinterpret_cast<v4u *>(nbase + xlds[b] + 16) = od;
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int a = 0; a < TN; ++a)
                    asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0"
                                 : "+a"(acc[a][b])
                                 : "v"(par ? wo[a] : we[a]), "v"(fx[step & 1][b]));
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        __syncthreads();
    };

    using PF0 = std::integral_constant<int, 0>;
    using PF1 = std::integral_constant<int, 1>;
    using PF2 = std::integral_constant<int, 2>;
    const bool ragged = nchunks != nfull;
    // prologue: chunk 0 into registers / LDS
    if (nfull > 0) {
        load_w(PF1{}, 0, 0);
        load_w(PF1{}, 1, 0);
        load_x(PF1{}, 0);
    } else {
        load_w(PF2{}, 0, 0);
        load_w(PF2{}, 1, 0);
        load_x(PF2{}, 0);
    }
    store_x(0);
    __syncthreads();
    uint32_t c = 0;
    for (; c + 1 < nfull; ++c) body(PF1{}, c);       // next chunk is a full one
    if (c + 1 < nchunks) {                           // next (last) chunk is ragged
        body(PF2{}, c);
        ++c;
    }
    if (c < nchunks) body(PF0{}, c);                 // last chunk: nothing to fetch
    (void)ragged;
    // the MFMAs above are opaque to the compiler's hazard tracking: let the last ones retire
    // before the accumulators are read
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

    const bool vec_ok = (EPI < 0) ? (p.N % 4 == 0 && reinterpret_cast<uintptr_t>(p.C) % 16 == 0)
                                  : (p.N % 4 == 0 && reinterpret_cast<uintptr_t>(p.y) % 8 == 0);
#pragma unroll
    for (int b = 0; b < TM; ++b)
#pragma unroll
        for (int a = 0; a < TN; ++a) {
            v4i v = acc[a][b];
#pragma unroll
            for (int r = 0; r < 4; ++r) v[r] >>= 8;
            store_quad<EPI, BIAS>(p, m0 + b * 16 + l16, n0 + wave * WN + a * 16 + g * 4, v, vec_ok);
        }
}

// ---------------------------------------------------------------------------------
// skinny kernel (M <= 16)
// ---------------------------------------------------------------------------------
// Workgroup = WAVES wavefronts, 16 output columns.  Wavefront w owns the k range
// [w*kw, (w+1)*kw) with kw = ceil(K/64/WAVES)*64 elements, walked in steps of 128 k (64 B
// per row): lane (l16, g) loads bytes [g*16, g*16+16) of the 64-byte segment of weight
// row n0+l16 and of activation row l16, expands both and issues two MFMAs (even k, odd k).
constexpr int kSkinnyUnroll = 8;  // 128-bit loads in flight per operand per lane

template <int WAVES, int EPI, bool BIAS>
__global__ __launch_bounds__(WAVES * 64) void gemm_s4_skinny_kernel(GemmParams p)
{
    __shared__ v4i part[WAVES][64];
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u, wave = tid >> 6;
    const uint32_t l16 = lane & 15u, g = lane >> 4;
    const uint32_t n0 = blockIdx.x * 16;
    const uint32_t kbytes = p.K >> 1;
    const uint32_t segs = kbytes / 64 + ((kbytes % 64) ? 1 : 0);  // 64-byte segments per row
    const uint32_t per_wave = (segs + WAVES - 1) / WAVES;
    const uint32_t seg_begin = wave * per_wave;
    const uint32_t seg_end = min(seg_begin + per_wave, segs);

    const uint32_t wrow = min(n0 + l16, p.N - 1);
    const bool xrow_ok = l16 < p.M;
    const uint8_t *wsrc = p.B + (uint64_t)wrow * kbytes + g * 16;
    const uint8_t *xsrc = p.A + (uint64_t)(xrow_ok ? l16 : 0) * kbytes + g * 16;

    v4i acc = v4i{0, 0, 0, 0};
    for (uint32_t s0 = seg_begin; s0 < seg_end; s0 += kSkinnyUnroll) {
        v4u w[kSkinnyUnroll], x[kSkinnyUnroll];
#pragma unroll
        for (int u = 0; u < kSkinnyUnroll; ++u) {
            const uint32_t off = (s0 + u) * 64;
            const bool ok = (s0 + u) < seg_end && off + g * 16 < kbytes;
            w[u] = ok ? __builtin_nontemporal_load(reinterpret_cast<const v4u *>(wsrc + off)) : v4u{0u, 0u, 0u, 0u};
            x[u] = (ok && xrow_ok) ? *reinterpret_cast<const v4u *>(xsrc + off) : v4u{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int u = 0; u < kSkinnyUnroll; ++u) {
            v4u we, wo, xe, xo;
            expand_nibbles(w[u], we, wo);
            expand_nibbles(x[u], xe, xo);
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(v4i, we), __builtin_bit_cast(v4i, xe),
                                                        acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(v4i, wo), __builtin_bit_cast(v4i, xo),
                                                        acc, 0, 0, 0);
        }
    }

    if (WAVES > 1) {
        part[wave][lane] = acc;
        __syncthreads();
        if (wave != 0) return;
#pragma unroll
        for (int w = 1; w < WAVES; ++w) {
            const v4i o = part[w][lane];
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[r] += o[r];
        }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) acc[r] >>= 8;
    const bool vec_ok = (EPI < 0) ? (p.N % 4 == 0 && reinterpret_cast<uintptr_t>(p.C) % 16 == 0)
                                  : (p.N % 4 == 0 && reinterpret_cast<uintptr_t>(p.y) % 8 == 0);
    store_quad<EPI, BIAS>(p, l16, n0 + g * 4, acc, vec_ok);
}

// ---------------------------------------------------------------------------------
// dispatch
// ---------------------------------------------------------------------------------
template <int EPI, bool BIAS>
static void launch_epi(GemmParams &p, hipStream_t stream)
{
    if (p.M <= 16) {
        const dim3 grid((p.N + 15) / 16);
        const uint32_t segs = (p.K / 2 + 63) / 64;
        // enough wavefronts per workgroup that each walks about one unrolled step of K
        if (segs <= 4 * kSkinnyUnroll)
            hipLaunchKernelGGL((gemm_s4_skinny_kernel<4, EPI, BIAS>), grid, dim3(256), 0, stream, p);
        else if (segs <= 8 * kSkinnyUnroll)
            hipLaunchKernelGGL((gemm_s4_skinny_kernel<8, EPI, BIAS>), grid, dim3(512), 0, stream, p);
        else
            hipLaunchKernelGGL((gemm_s4_skinny_kernel<16, EPI, BIAS>), grid, dim3(1024), 0, stream, p);
        return;
    }
    // largest tile that still yields at least one workgroup per CU (256 CUs); small
    // problems take the small tile to spread over the chip.
    auto tiles = [&](uint32_t bm, uint32_t bn) { return ((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn); };
    static const int variant = getenv("DUQ_GEMM_VARIANT") ? atoi(getenv("DUQ_GEMM_VARIANT")) : 1;
    if (variant == 1 && tiles(128, 256) >= 128 && p.M > 64) {
        p.tiles_m = (p.M + 127) / 128;
        p.tiles_n = (p.N + 255) / 256;
        hipLaunchKernelGGL((gemm_s4_stream_kernel<8, 4, EPI, BIAS>), dim3(p.tiles_m * p.tiles_n), dim3(256), 0,
                           stream, p);
    } else if (tiles(128, 256) >= 256 && p.M > 64) {
        p.tiles_m = (p.M + 127) / 128;
        p.tiles_n = (p.N + 255) / 256;
        hipLaunchKernelGGL((gemm_s4_tile_kernel<128, 256, EPI, BIAS>), dim3(p.tiles_m * p.tiles_n), dim3(256), 0,
                           stream, p);
    } else if (tiles(128, 128) >= 256 && p.M > 64) {
        p.tiles_m = (p.M + 127) / 128;
        p.tiles_n = (p.N + 127) / 128;
        hipLaunchKernelGGL((gemm_s4_tile_kernel<128, 128, EPI, BIAS>), dim3(p.tiles_m * p.tiles_n), dim3(256), 0,
                           stream, p);
    } else {
        p.tiles_m = (p.M + 63) / 64;
        p.tiles_n = (p.N + 63) / 64;
        hipLaunchKernelGGL((gemm_s4_tile_kernel<64, 64, EPI, BIAS>), dim3(p.tiles_m * p.tiles_n), dim3(256), 0,
                           stream, p);
    }
}

int launch_gemm_s4(const uint8_t *A, const uint8_t *B, uint32_t M, uint32_t N, uint32_t K, int32_t *out_acc,
                   const Epilogue *epi, uint16_t *y, hipStream_t stream)
{
    if (M == 0 || N == 0) return 0;
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
        launch_epi<-1, false>(p, stream);
    } else {
        const bool bias = epi->bias != nullptr;
#define DUQ_GEMM(MODE)                             \
    case MODE:                                     \
        if (bias)                                  \
            launch_epi<MODE, true>(p, stream);     \
        else                                       \
            launch_epi<MODE, false>(p, stream);    \
        break;
        switch (epi->mode) {
            DUQ_GEMM(0)
            DUQ_GEMM(1)
            DUQ_GEMM(2)
            DUQ_GEMM(3)
        default:
            return (int)hipErrorInvalidValue;
        }
#undef DUQ_GEMM
    }
    return (int)hipGetLastError();
}

}  // namespace duq
