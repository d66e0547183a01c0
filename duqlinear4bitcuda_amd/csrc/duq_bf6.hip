// The same int4 x int4 GEMM on the 6-bit floating point matrix path of gfx950.
//
// Every int4 value -8..7 is exactly an E3M2 ("bf6") number, every product of two of them is
// an integer of at most 7 bits, and the float32 accumulator of v_mfma_f32_16x16x128_f8f6f4
// holds every integer below 2^24 exactly.  |C| <= 64*K < 2^24 for K <= 131008 (the bound of
// the integer kernels), all partial sums are integers below 2^24 whatever the order, so the
// float32 result converted back to int32 is the integer result bit for bit.  The instruction
// runs at twice the rate of the i8 MFMA and the operands need no expansion in the loop.
//
// Operands are "shadows" of the packed-int4 tensors, made once (weights) or by the quantizer
// (activations).  A block is 32 consecutive k of one row: 32 codes x 6 bits = 24 bytes, as
// v_cvt_scalef32_pk32_bf6_f16 writes them; it is kept as a 16-byte part and an 8-byte part
// so that every load is naturally aligned.
//   activation shadow  [M][K/32 x 16 B | K/32 x 8 B]      (row-major, two planes per row)
//   weight shadow      [ceil(N/32)][K/128][3][64 lanes x 16 B]
//                      lane l of a (pair of 16-row tiles, 128-k step) holds the blocks of row l % 16,
//                      k-block l / 16 of either tile: 12 dwords [tile 2p | tile 2p+1], cut into three
//                      16-byte pieces; piece r of all lanes is one contiguous kilobyte.  Three 128-bit
//                      loads bring the two MFMA operands into twelve consecutive registers, which the
//                      kernel pins (mfma_pinned) so that the loads write them in place: three memory
//                      instructions per two fragments instead of four (a 128-bit and a 64-bit load per
//                      fragment), without a register move.  An odd last tile is paired with zeros.
// K % 128 == 0 and N % 16 == 0.
//
// Kernel: tile 128 (M) x 256 (N) per workgroup, 4 wavefronts side by side along N (128 x 64
// each: 8 x 4 MFMA tiles, 128 accumulator registers).  Weights go global -> registers (a ring
// of four 128-k steps), activations global -> registers -> LDS (three buffers of 256 k, one
// barrier per buffer) -> fragments read two MFMA groups ahead.  The weight operand is the
// MFMA "A" side, so a lane ends up with four consecutive output columns of one row.
#include "duq_epilogue.h"
#include "duq_launch.h"
#include "duq_tiles.h"
#include <type_traits>

namespace duq {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v6i __attribute__((ext_vector_type(6)));
typedef int v12i __attribute__((ext_vector_type(12)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v32h __attribute__((ext_vector_type(32)));

// ---------------------------------------------------------------------------------
// weight shadow
// ---------------------------------------------------------------------------------
// 32 signed nibbles (16 bytes, element 2j in the low nibble of byte j) -> one bf6 block.
// Position 8d + 2i + h of the block holds nibble i + 4h of word d (the order the quantizer
// kernels produce cheaply); both operands use it, and the sum over k does not care.
__device__ __forceinline__ v6i bf6_block_from_nibbles(const v4u w)
{
    v32h f;
#pragma unroll
    for (int pos = 0; pos < 32; ++pos) {
        const int d = pos >> 3, e = ((pos & 7) >> 1) + 4 * (pos & 1);
        const int v = ((int)(w[d] << (28 - 4 * e))) >> 28;
        f[pos] = (f16)(float)v;
    }
    return __builtin_bit_cast(v6i, __builtin_amdgcn_cvt_scalef32_pk32_bf6_f16(f, 1.0f));
}

// Layout: for every pair of 16-row tiles and every 128-k step, 3072 bytes.  Lane l = (row l % 16, k-block l / 16) owns
// one block (24 bytes = 6 dwords) of either tile; its 12 dwords [tile 2p | tile 2p+1] are cut into three 16-byte
// pieces, and piece r of all 64 lanes forms run r (1 KB): three 128-bit loads bring two MFMA operands into twelve
// consecutive registers.  An odd last tile is paired with zeros.
__global__ __launch_bounds__(256) void weight_shadow_kernel(const uint8_t *w, uint32_t N, uint32_t K, uint8_t *out)
{
    const uint32_t ksteps = K / 128, tiles = N / 16;
    const uint64_t total = (uint64_t)((tiles + 1) / 2) * ksteps * 64;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (uint64_t)gridDim.x * blockDim.x) {
        const uint32_t lane = (uint32_t)(i & 63u);
        const uint64_t ps = i >> 6;  // pair * ksteps + step
        const uint32_t step = (uint32_t)(ps % ksteps), pair = (uint32_t)(ps / ksteps);
        const uint32_t kb = step * 4 + (lane >> 4);
        v6i f[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint32_t tile = pair * 2 + h, n = tile * 16 + (lane & 15u);
            f[h] = v6i{0, 0, 0, 0, 0, 0};
            if (tile < tiles) f[h] = bf6_block_from_nibbles(*reinterpret_cast<const v4u *>(w + (uint64_t)n * (K / 2) + kb * 16));
        }
        uint8_t *dst = out + ps * 3072 + lane * 16;
        *reinterpret_cast<v4i *>(dst) = v4i{f[0][0], f[0][1], f[0][2], f[0][3]};
        *reinterpret_cast<v4i *>(dst + 1024) = v4i{f[0][4], f[0][5], f[1][0], f[1][1]};
        *reinterpret_cast<v4i *>(dst + 2048) = v4i{f[1][2], f[1][3], f[1][4], f[1][5]};
    }
}

int launch_weight_shadow_bf6(const uint8_t *w, uint32_t N, uint32_t K, uint8_t *out, hipStream_t stream)
{
    const uint64_t total = (uint64_t)((N / 16 + 1) / 2) * (K / 128) * 64;
    if (total == 0) return 0;
    const uint32_t blocks = (uint32_t)std::min<uint64_t>((total + 255) / 256, 1u << 16);
    hipLaunchKernelGGL(weight_shadow_kernel, dim3(blocks), dim3(256), 0, stream, w, N, K, out);
    return (int)hipGetLastError();
}

// activation shadow from packed nibbles (the quantizers write it directly; this is the
// stand-alone conversion for tensors quantized elsewhere)
__global__ __launch_bounds__(256) void activation_shadow_kernel(const uint8_t *q, uint32_t M, uint32_t K, uint8_t *out)
{
    const uint32_t nblk = K / 32;
    const uint64_t total = (uint64_t)M * nblk;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (uint64_t)gridDim.x * blockDim.x) {
        const uint32_t b = (uint32_t)(i % nblk);
        const uint64_t m = i / nblk;
        const v4u raw = *reinterpret_cast<const v4u *>(q + m * (K / 2) + b * 16);
        const v6i f = bf6_block_from_nibbles(raw);
        uint8_t *row = out + m * (uint64_t)nblk * 24;
        *reinterpret_cast<v4i *>(row + b * 16) = v4i{f[0], f[1], f[2], f[3]};
        *reinterpret_cast<v2i *>(row + (uint64_t)nblk * 16 + b * 8) = v2i{f[4], f[5]};
    }
}

int launch_activation_shadow_bf6(const uint8_t *q, uint32_t M, uint32_t K, uint8_t *out, hipStream_t stream)
{
    const uint64_t total = (uint64_t)M * (K / 32);
    if (total == 0) return 0;
    const uint32_t blocks = (uint32_t)std::min<uint64_t>((total + 255) / 256, 1u << 16);
    hipLaunchKernelGGL(activation_shadow_kernel, dim3(blocks), dim3(256), 0, stream, q, M, K, out);
    return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------------
// GEMM
// ---------------------------------------------------------------------------------
// Workgroup barrier that waits for this wavefront's LDS traffic only.  __syncthreads() also
// drains the vector memory counter, which here would wait for the weight and activation
// prefetches issued just before it (a full memory latency per chunk).
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Cache policy of the output stores: 2 = non-temporal.  The output is written once and read by nobody in this
// launch; streamed past the L2 it leaves the operand panels there and the launch ends sooner (measured at
// M = 2048, N = K = 4096: 21.8 against 23.0 us; same bits).
#ifndef DUQ_BF6_STORE_AUX
#define DUQ_BF6_STORE_AUX 2
#endif

#ifndef DUQ_BF6_COST64
#define DUQ_BF6_COST64 0.68f
#endif
#ifndef DUQ_BF6_COST256
#define DUQ_BF6_COST256 1.78f
#endif
#ifndef DUQ_BF6_NARROW_MAX_TILES
#define DUQ_BF6_NARROW_MAX_TILES 128
#endif

// One MFMA on half h (0: registers 0..5, 1: registers 6..11) of weight pair tuple t, which lives in the twelve
// registers v[128 + 12*t .. 139 + 12*t].  Naming the registers pins the tuple, so that the three 128-bit loads that
// fill it write them in place and the two operands are its halves: no register moves, which an opaque MFMA would
// need wait states behind (a "v" operand cannot name half of a tuple).  t and h are constants after unrolling; the
// switch folds to one statement.
#define DUQ_PIN(T, A0, A1, B0, B1)                                                                                     \
    case 2 * T:                                                                                                       \
        asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, v[" #A0 ":" #A1 "], %1, %0 cbsz:3 blgp:3"                        \
                     : "+a"(acc)                                                                                       \
                     : "v"(x), "{v[" #A0 ":" #B1 "]}"(w));                                                             \
        break;                                                                                                        \
    case 2 * T + 1:                                                                                                   \
        asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, v[" #B0 ":" #B1 "], %1, %0 cbsz:3 blgp:3"                        \
                     : "+a"(acc)                                                                                       \
                     : "v"(x), "{v[" #A0 ":" #B1 "]}"(w));                                                             \
        break;
// BASE: first register of the ring (chosen per kernel variant so that the ring ends where the variant's register
// count ends: the tuples are pinned, everything else is the compiler's).
template <int BASE>
__device__ __forceinline__ void mfma_pinned(int t, int h, v4f &acc, const v12i &w, const v6i &x)
{
    static_assert(BASE == 64 || BASE == 96 || BASE == 128 || BASE == 160, "ring base registers with a table below");
    if (BASE == 64) {  // 4 tuples (64 x 128 tiles)
        switch (2 * t + h) {
        DUQ_PIN(0, 64, 69, 70, 75)
        DUQ_PIN(1, 76, 81, 82, 87)
        DUQ_PIN(2, 88, 93, 94, 99)
        DUQ_PIN(3, 100, 105, 106, 111)
        default: __builtin_unreachable();
        }
    } else if (BASE == 96) {
        switch (2 * t + h) {
        DUQ_PIN(0, 96, 101, 102, 107)
        DUQ_PIN(1, 108, 113, 114, 119)
        DUQ_PIN(2, 120, 125, 126, 131)
        DUQ_PIN(3, 132, 137, 138, 143)
        DUQ_PIN(4, 144, 149, 150, 155)
        DUQ_PIN(5, 156, 161, 162, 167)
        DUQ_PIN(6, 168, 173, 174, 179)
        DUQ_PIN(7, 180, 185, 186, 191)
        default: __builtin_unreachable();
        }
    } else if (BASE == 128) {
        switch (2 * t + h) {
        DUQ_PIN(0, 128, 133, 134, 139)
        DUQ_PIN(1, 140, 145, 146, 151)
        DUQ_PIN(2, 152, 157, 158, 163)
        DUQ_PIN(3, 164, 169, 170, 175)
        DUQ_PIN(4, 176, 181, 182, 187)
        DUQ_PIN(5, 188, 193, 194, 199)
        DUQ_PIN(6, 200, 205, 206, 211)
        DUQ_PIN(7, 212, 217, 218, 223)
        default: __builtin_unreachable();
        }
    } else {
        switch (2 * t + h) {
        DUQ_PIN(0, 160, 165, 166, 171)
        DUQ_PIN(1, 172, 177, 178, 183)
        DUQ_PIN(2, 184, 189, 190, 195)
        DUQ_PIN(3, 196, 201, 202, 207)
        DUQ_PIN(4, 208, 213, 214, 219)
        DUQ_PIN(5, 220, 225, 226, 231)
        DUQ_PIN(6, 232, 237, 238, 243)
        DUQ_PIN(7, 244, 249, 250, 255)
        default: __builtin_unreachable();
        }
    }
}
#undef DUQ_PIN

// The first 56 bytes (through epi.mode) reach the kernel in registers (DUQ_HEAD_DECL / with_head).
struct Bf6Params {
    const uint8_t *X;  // activation shadow
    const uint8_t *W;  // weight shadow
    uint32_t M, N, K;
    uint32_t tiles_m;
    uint16_t *y;
    uint32_t tiles_n;
    Epilogue epi;
    // epilogue mode 5 only: the packed-int4 operands the shadows were made from (the first eight bytes of every row
    // are read: the codes of input columns 0..9)
    const uint8_t *xq;
    const uint8_t *wq;
};
static_assert(offsetof(Bf6Params, epi) + 8 == kHeadBytes, "the fields delivered in registers");

// TMI = 8: 128-row tiles.  TMI = 4: 64-row tiles for problems that would leave most CUs without a 128-row tile
// (half the MFMAs for the same weight traffic, but twice the workgroups).  TMI = 16: 256-row tiles for problems
// with at least one such tile per CU: the same weight traffic feeds twice the MFMAs, which takes the kernel off
// the L2 -> CU limit that bounds the smaller tiles; all 256 AGPRs hold accumulators, an activation chunk is one
// 128-k step (three buffers of two steps would not fit in LDS) and the epilogue parameters are fetched after the loop.
template <int TMI, int TNI, int EPI, bool BIAS>
__global__ __launch_bounds__(256) void gemm_bf6_kernel(DUQ_HEAD_DECL, Bf6Params tail)
{
    Bf6Params p = with_head(tail, DUQ_HEAD_USE);
    to_global(p.X);
    to_global(p.W);
    to_global(p.y);
    static_assert(TMI == 16 || TMI == 8 || TMI == 4, "16-row MFMA tiles per wavefront along M");
    // TNI = 16 x 16 MFMA tiles per wavefront along N: BM rows x 64 columns (TNI = 4), or BM x 32 (TNI = 2, with
    // 64-row tiles only: twice the workgroups for problems that leave CUs without a 64 x 256 tile)
    static_assert(TNI == 4 || (TNI == 2 && TMI == 4), "column tiles per wavefront");
    constexpr int BM = 16 * TMI, BN = 64 * TNI;
    constexpr int CH = TMI == 16 ? 1 : 2;  // 128-k steps per activation chunk
    constexpr int NPH = 4 / CH;            // chunk bodies per turn of the weight ring
    // 16-byte activation pieces per thread and chunk: plane 0 (4*CH per row), plane 1 (2*CH per row)
    constexpr int NX0 = BM * 4 * CH / 256, NX1 = BM * 2 * CH / 256, NXP = NX0 + NX1;
    // LDS bytes per row: the 16-byte (8-byte) parts of the 4*CH blocks of a chunk + 16 bytes of padding, which
    // makes the fragment reads of 16 rows conflict-free
    constexpr uint32_t kP0Stride = 64 * CH + 16, kP1Stride = 32 * CH + 16;
    constexpr uint32_t kP1Base = BM * kP0Stride;
    constexpr uint32_t kBuf = BM * (kP0Stride + kP1Stride);
    constexpr uint32_t kYStride = 32 * TNI + 16;  // bytes per staged output row: 16*TNI binary16 + pad
    constexpr uint32_t kLds = 3 * kBuf > 4 * BM * kYStride ? 3 * kBuf : 4 * BM * kYStride;
    constexpr bool LATE_PARAMS = TMI == 16;
    constexpr int MODE = EPI;

    __shared__ __attribute__((aligned(16))) uint8_t lds[kLds];
    // dual-uniform row-sum epilogue (EPI 5): its parameters, eight words per column of the tile and per row, fetched
    // by the first BN / BM threads before the loop and read back from here after it (the records of the integer
    // kernel's epilogue, gemm_s4_stream_kernel)
    //   column: wlo, whi (first eight bytes of the packed weight row), s1 | s2 << 16, z1, z2, adj1, adj2, bias
    //   row   : xlo, xhi & 0xFF (first ten codes of the packed activation row), float(s), z, rx - rxl, rxl
    __shared__ __attribute__((aligned(16))) uint32_t dpar[EPI == 5 ? (BN + BM) * 8 : 4];
    __shared__ uint32_t dwide;  // EPI 5: non-zero when a factor of the corrections leaves the signed 24-bit range

    uint32_t tile_m, tile_n;
    tile_of_block(blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u, wave = tid >> 6;
    const uint32_t l16 = lane & 15u, kb = lane >> 4;
    if constexpr (EPI == 5) {
        const uint32_t kbytes = p.K >> 1;
        if (tid == 0) dwide = 0;
        __syncthreads();
        bool wide = false;
        for (uint32_t i = tid; i < (uint32_t)BN; i += 256) {
            const uint32_t n = min(n0 + i, p.N - 1);
            const v2u head = *reinterpret_cast<const v2u *>(p.wq + (uint64_t)n * kbytes);
            uint32_t *d = dpar + i * 8;
            d[0] = head[0];
            d[1] = head[1];
            d[2] = (uint32_t)p.epi.s_col_1[n] | ((uint32_t)p.epi.s_col_2[n] << 16);
            d[3] = (uint32_t)rint_i32((float)bits_to_f16(p.epi.z_col_1[n]));
            d[4] = (uint32_t)rint_i32((float)bits_to_f16(p.epi.z_col_2[n]));
            d[5] = (uint32_t)p.epi.rs_col[n];
            d[6] = (uint32_t)p.epi.rs_col_2[n];
            d[7] = BIAS ? (uint32_t)p.epi.bias[n] : 0u;
            wide = wide || !(fits_i24(d[3]) && fits_i24(d[4]) && fits_i24(d[5]) && fits_i24(d[6]));
        }
        for (uint32_t i = tid; i < (uint32_t)BM; i += 256) {
            const uint32_t m = min(m0 + i, p.M - 1);
            const v2u head = *reinterpret_cast<const v2u *>(p.xq + (uint64_t)m * kbytes);
            const uint32_t xlo = head[0], xhi = head[1] & 0xFFu;  // input columns 0..7 and 8, 9
            const uint32_t rxl = dual_head_sum(xlo, xhi);
            uint32_t *d = dpar + (BN + i) * 8;
            d[0] = xlo;
            d[1] = xhi;
            d[2] = __builtin_bit_cast(uint32_t, (float)bits_to_f16(p.epi.s_row[m]));
            d[3] = (uint32_t)rint_i32((float)bits_to_f16(p.epi.z_row[m]));
            d[4] = (uint32_t)p.epi.rs_row[m] - rxl;
            d[5] = rxl;
            wide = wide || !(fits_i24(d[3]) && fits_i24(d[4]));
        }
        if (wide) dwide = 1;  // (same value from every writer)
        // (the barriers of the main loop order these writes before the epilogue's reads)
    }
    const uint32_t nblk = p.K / 32;
    const uint32_t row_bytes = nblk * 24, p1off = nblk * 16;
    const uint32_t ksteps = p.K / 128;
    const uint32_t nchunks = (ksteps + CH - 1) / CH;

    const uint32_t wpairs = (min(p.N - n0, (uint32_t)BN) / 16 + 1) / 2;  // pairs of 16-row weight tiles in this tile
    const __amdgpu_buffer_rsrc_t rW =
        make_rsrc(p.W + (uint64_t)(n0 / 32) * ksteps * 3072, wpairs * ksteps * 3072);
    const __amdgpu_buffer_rsrc_t rX =
        make_rsrc(p.X + (uint64_t)m0 * row_bytes, min(p.M - m0, (uint32_t)BM) * row_bytes);
    const __amdgpu_buffer_rsrc_t rNone = make_rsrc(p.X, 0);  // every read returns zero

    // weight fragments (2*pi, 2*pi + 1) of step g: 3072 bytes at ((wave*NP + pi) * ksteps + g) * 3072, three 16-byte
    // parts per lane (12 consecutive registers: two MFMA operands).  The scalar offset is not part of the hardware
    // range check: pairs past N sit in the vector offset, steps past K switch to the empty descriptor.
    constexpr int NP = TNI / 2;
    constexpr int kRingBase = TNI == 2 ? 64 : (TMI == 16 ? 160 : (TMI == 4 ? 96 : 128));
    uint32_t wv[NP];
#pragma unroll
    for (int pi = 0; pi < NP; ++pi)
        wv[pi] = wave * NP + pi < wpairs ? (wave * NP + pi) * ksteps * 3072 + lane * 16 : kOobOffset;
    // part 0..2 of the pair's twelve registers
    auto load_w = [&](v12i &dst, int pi, int part, uint32_t g, __amdgpu_buffer_rsrc_t r) {
        const v4i a = __builtin_bit_cast(
            v4i, __builtin_amdgcn_raw_buffer_load_b128(r, (int)(wv[pi] == kOobOffset ? kOobOffset : wv[pi] + part * 1024),
                                                       (int)(g * 3072), 0));
        dst[4 * part + 0] = a[0], dst[4 * part + 1] = a[1], dst[4 * part + 2] = a[2], dst[4 * part + 3] = a[3];
    };

    // activation pieces of a chunk (256 k = 8 blocks): NX0 of plane 0 and NX1 of plane 1 per thread
    uint32_t xoff[NXP], xlds[NXP];
#pragma unroll
    for (int j = 0; j < NX0; ++j) {
        const uint32_t row = tid / (4 * CH) + j * (256 / (4 * CH)), piece = tid % (4 * CH);
        xoff[j] = row * row_bytes + piece * 16;
        xlds[j] = row * kP0Stride + piece * 16;
    }
#pragma unroll
    for (int j = 0; j < NX1; ++j) {
        const uint32_t row = tid / (2 * CH) + j * (256 / (2 * CH)), piece = tid % (2 * CH);
        xoff[NX0 + j] = row * row_bytes + p1off + piece * 16;
        xlds[NX0 + j] = kP1Base + row * kP1Stride + piece * 16;
    }
    // piece j of chunk c.  The chunk offset rides in the vector offset so that the range check sees it: when
    // K is an odd number of steps the last chunk's second half reads the next row (unused) or, in the last
    // row, past the descriptor (zero).
    auto load_x = [&](v4u &dst, int j, uint32_t c, __amdgpu_buffer_rsrc_t r) {
        dst = buf_load16(r, xoff[j] + (j < NX0 ? c * (64 * CH) : c * (32 * CH)), 0);
    };

    // fragment of rows mi*16 + l16, k-step s of a chunk: plane 0 + mi*16*kP0Stride + s*64, plane 1 + ... + s*32
    const uint32_t frag0 = l16 * kP0Stride + kb * 16, frag1 = kP1Base + l16 * kP1Stride + kb * 8;

    v12i wf[4][NP];   // weight fragment pairs [ring slot][pair of column tiles], pinned to v[kRingBase + 12 * (slot * NP + pi) ..]
    v6i xf[4];        // activation fragments, ring over mi
    v4u xreg[NXP];
    v4f acc[TMI][TNI];
#pragma unroll
    for (int a = 0; a < TMI; ++a)
#pragma unroll
        for (int b = 0; b < TNI; ++b) acc[a][b] = v4f{0.f, 0.f, 0.f, 0.f};

    auto read_x0 = [&](v6i &dst, uint32_t buf, int mi, int s) {
        const v4i a = *reinterpret_cast<const v4i *>(lds + buf + frag0 + mi * 16 * kP0Stride + s * 64);
        dst[0] = a[0], dst[1] = a[1], dst[2] = a[2], dst[3] = a[3];
    };
    auto read_x1 = [&](v6i &dst, uint32_t buf, int mi, int s) {
        const v2i b = *reinterpret_cast<const v2i *>(lds + buf + frag1 + mi * 16 * kP1Stride + s * 32);
        dst[4] = b[0], dst[5] = b[1];
    };

    // ---- prologue: weights of steps 0..3, activations of chunks 0 and 1 -> LDS, chunk 2 -> registers.  Issued
    // in the order of first use, so that the wait for the two activation chunks (vector memory waits are in
    // order) leaves the weights of steps 1..3 in flight: all 256 workgroups start together and their first
    // ~170 KB each are bound by the L2 -> CU rate, not by latency.
    v4u x1[NXP];
#pragma unroll
    for (int j = 0; j < NXP; ++j) load_x(xreg[j], j, 0, rX);
#pragma unroll
    for (int pi = 0; pi < NP; ++pi)
#pragma unroll
        for (int part = 0; part < 3; ++part) load_w(wf[0][pi], pi, part, 0, rW);
#pragma unroll
    for (int j = 0; j < NXP; ++j) load_x(x1[j], j, 1, 1 < nchunks ? rX : rNone);
#pragma unroll
    for (int g = 1; g < 4; ++g)
#pragma unroll
        for (int pi = 0; pi < NP; ++pi)
#pragma unroll
            for (int part = 0; part < 3; ++part) load_w(wf[g][pi], pi, part, g, (uint32_t)g < ksteps ? rW : rNone);
#pragma unroll
    for (int j = 0; j < NXP; ++j) *reinterpret_cast<v4u *>(lds + xlds[j]) = xreg[j];
#pragma unroll
    for (int j = 0; j < NXP; ++j) *reinterpret_cast<v4u *>(lds + kBuf + xlds[j]) = x1[j];
#pragma unroll
    for (int j = 0; j < NXP; ++j) load_x(xreg[j], j, 2, 2 < nchunks ? rX : rNone);
    lds_barrier();
#pragma unroll
    for (int mi = 0; mi < 2; ++mi) {
        read_x0(xf[mi], 0, mi, 0);
        read_x1(xf[mi], 0, mi, 0);
    }

    // ---- epilogue parameters: fetched now so that their latency hides behind the main loop (after the loop for
    // the 256-row tile, whose loop has no registers to spare)
    const Epilogue &e = p.epi;
    v2u raw_s1[TNI], raw_z1[TNI], raw_s2[TNI], raw_z2[TNI], raw_bias[TNI];
    v4i raw_rs[TNI];
    RowEpi rowp[TMI];
    auto load_params = [&]() {
        if constexpr (EPI == 5) return;  // staged in LDS above
#pragma unroll
        for (int mi = 0; mi < TMI; ++mi) rowp[mi] = load_row<MODE == 5 ? 0 : MODE>(e, min(m0 + mi * 16 + l16, p.M - 1));
#pragma unroll
        for (int ni = 0; ni < TNI; ++ni) {
            const uint32_t nq = min(n0 + wave * (16 * TNI) + ni * 16 + kb * 4, p.N - 4);
            raw_s1[ni] = *reinterpret_cast<const v2u *>(e.s_col_1 + nq);
            if (MODE == 1 || MODE == 3 || MODE == 4) raw_z1[ni] = *reinterpret_cast<const v2u *>(e.z_col_1 + nq);
            if (MODE == 4) raw_rs[ni] = *reinterpret_cast<const v4i *>(e.rs_col + nq);
            if (MODE >= 2 && MODE != 4) raw_s2[ni] = *reinterpret_cast<const v2u *>(e.s_col_2 + nq);
            if (MODE == 3) raw_z2[ni] = *reinterpret_cast<const v2u *>(e.z_col_2 + nq);
            if (BIAS) raw_bias[ni] = *reinterpret_cast<const v2u *>(e.bias + nq);
        }
    };
    if (!LATE_PARAMS) load_params();

    // One chunk = CH 128-k steps.  PH = position of the chunk in a turn of the weight ring: its steps use ring
    // slots CH*PH ..; a slot is refilled (with the step four ahead) during the step after its use.
    auto chunk = [&](auto ph, uint32_t c, uint32_t cur, uint32_t nxt, uint32_t nx2) {
        constexpr int PH = decltype(ph)::value;
        // Side work is spread one instruction per MFMA: the loop is bound by the issue rate of its single
        // wavefront per SIMD, and a slot that holds more than about 12 cycles of other work stalls the matrix pipe.
        const __amdgpu_buffer_rsrc_t rXc = c + 3 < nchunks ? rX : rNone;
#pragma unroll
        for (int s = 0; s < CH; ++s) {
            const int slot = CH * PH + s;
            const int prev = (slot + 3) & 3;          // slot of the step before this one
            const uint32_t gprev = CH * c + s - 1 + 4;  // the step that slot receives now
            const __amdgpu_buffer_rsrc_t rG = gprev < ksteps ? rW : rNone;
#pragma unroll
            for (int mi = 0; mi < TMI; ++mi) {
#pragma unroll
                for (int ni = 0; ni < TNI; ++ni) {
                    // The operands are written by loads only (the compiler waits for those).  A register move
                    // placed right in front of this opaque statement would need wait states the compiler
                    // cannot know of; the generated loop has none, and the bit-exact parity tests would show one.
                    mfma_pinned<kRingBase>(slot * NP + ni / 2, ni & 1, acc[mi][ni], wf[slot][ni / 2], xf[mi & 3]);
                    __builtin_amdgcn_sched_barrier(0);
                    // ---- side work in the shadow of this MFMA
                    if (ni < 2) {  // activation fragment two groups ahead
                        const int nm = (mi + 2) & (TMI - 1), ns = mi + 2 < TMI ? s : s + 1;
                        const uint32_t buf = ns < CH ? cur : nxt;
                        if (ni == 0)
                            read_x0(xf[nm & 3], buf, nm, ns % CH);
                        else
                            read_x1(xf[nm & 3], buf, nm, ns % CH);
                    }
                    // refill the previous step's slot: 3 * NP loads over the step (step 0 fetches step 3 again)
                    {
                        int widx = -1;  // which of the 3 * NP loads rides with this MFMA
                        if (TNI == 2) widx = mi < 2 ? mi * 2 + ni : -1;
                        if (TNI == 4 && TMI == 8) widx = ni == 2 ? mi : -1;
                        if (TNI == 4 && TMI == 4) widx = ni >= 2 ? mi * 2 + (ni - 2) : -1;
                        if (TNI == 4 && TMI == 16) widx = (ni == 2 && (mi & 1) == 0) ? mi / 2 : -1;
                        if (widx >= 0 && widx < 3 * NP) load_w(wf[prev][widx / 3], widx / 3, widx % 3, gprev, rG);
                    }
                    if (TNI == 2 && s == 1 && mi >= 2) {  // three activation pieces per chunk: store, then refetch
                        const int slot2 = (mi - 2) * 2 + ni;  // 0..3
                        if (slot2 < NXP) *reinterpret_cast<v4u *>(lds + nx2 + xlds[slot2]) = xreg[slot2];
                        if (slot2 >= 1 && slot2 <= NXP) load_x(xreg[slot2 - 1], slot2 - 1, c + 3, rXc);
                    }
                    // chunk c+2 -> its LDS buffer and, one group (one slot) later, chunk c+3 into the freed register
                    if (TNI == 4 && TMI <= 8 && s == 1 && mi < NXP && ni == (TMI == 8 ? 3 : 0))
                        *reinterpret_cast<v4u *>(lds + nx2 + xlds[mi]) = xreg[mi];
                    if (TNI == 4 && TMI <= 8 && s == 1 && ni == 1 && mi >= 1 && mi <= NXP)
                        load_x(xreg[mi - 1], mi - 1, c + 3, rXc);
                    if (TMI == 16 && (mi & 1) == 1 && (mi >> 1) < NXP) {
                        if (ni == 2) *reinterpret_cast<v4u *>(lds + nx2 + xlds[mi >> 1]) = xreg[mi >> 1];
                        if (ni == 3) load_x(xreg[mi >> 1], mi >> 1, c + 3, rXc);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        // the MFMAs are opaque to the compiler's hazard tracking: any accumulator copy it places
        // at a control-flow join must find them retired
        asm volatile("s_nop 15" ::: "memory");
        lds_barrier();
    };

    uint32_t cur = 0, nxt = kBuf, nx2 = 2 * kBuf;
    auto rotate = [&]() {
        const uint32_t t = cur;
        cur = nxt;
        nxt = nx2;
        nx2 = t;
    };
    using P0 = std::integral_constant<int, 0>;
    using P1 = std::integral_constant<int, 1>;
    using P2 = std::integral_constant<int, 2>;
    using P3 = std::integral_constant<int, 3>;
    uint32_t c = 0;
    // (no branch inside the loop: a path that skips a chunk would make the compiler count only that
    // path's loads when it waits for a fragment, and drain the prefetch ring every iteration)
    if (NPH == 2) {
        for (; c + 1 < nchunks; c += 2) {
            chunk(P0{}, c, cur, nxt, nx2);
            rotate();
            chunk(P1{}, c + 1, cur, nxt, nx2);
            rotate();
        }
        if (c < nchunks) chunk(P0{}, c, cur, nxt, nx2);
    } else {
        for (; c + 3 < nchunks; c += 4) {
            chunk(P0{}, c, cur, nxt, nx2);
            rotate();
            chunk(P1{}, c + 1, cur, nxt, nx2);
            rotate();
            chunk(P2{}, c + 2, cur, nxt, nx2);
            rotate();
            chunk(P3{}, c + 3, cur, nxt, nx2);
            rotate();
        }
        if (c < nchunks) {
            chunk(P0{}, c, cur, nxt, nx2);
            rotate();
            if (c + 1 < nchunks) {
                chunk(P1{}, c + 1, cur, nxt, nx2);
                rotate();
                if (c + 2 < nchunks) chunk(P2{}, c + 2, cur, nxt, nx2);
            }
        }
    }
    if (LATE_PARAMS) load_params();
    // the MFMAs above are opaque to the compiler's hazard tracking: let the last ones retire
    asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");

    // ---- epilogue: lane holds acc[mi][ni][r] = C[m = mi*16 + l16][n = ni*16 + 4*kb + r].  The
    // 128 x 64 fp16 tile of the wavefront goes through LDS so that global stores are whole
    // 128-byte lines.
    uint8_t *stage = lds + wave * (BM * kYStride);
    if constexpr (EPI == 5) {
        // every wavefront has passed the loop's last barrier: dpar is complete.  The staging area overlaps the
        // activation buffers that other wavefronts may still read in their last chunk: wait for them.
        __syncthreads();
        const bool wide = dwide != 0;
#pragma unroll
        for (int ni = 0; ni < TNI; ++ni) {
            const uint32_t ncol = ni * 16 + kb * 4;
            v4u c0[4], c1[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const uint32_t *d = dpar + (wave * (16 * TNI) + ncol + r) * 8;
                c0[r] = *reinterpret_cast<const v4u *>(d);
                c1[r] = *reinterpret_cast<const v4u *>(d + 4);
            }
#pragma unroll
            for (int mi = 0; mi < TMI; ++mi) {
                const uint32_t *d = dpar + (BN + mi * 16 + l16) * 8;
                const v4u r0 = *reinterpret_cast<const v4u *>(d);
                const v2u r1 = *reinterpret_cast<const v2u *>(d + 4);
                const uint32_t s_bits = r0[2];  // (a copy: a bit cast of a vector element would read element 0)
                const float sx = __builtin_bit_cast(float, s_bits);
                uint16_t out[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float s1 = (float)bits_to_f16((uint16_t)(c0[r][2] & 0xFFFFu)), s2 = (float)bits_to_f16((uint16_t)(c0[r][2] >> 16));
                    const f16 b = bits_to_f16((uint16_t)c1[r][3]);
                    const int a = (int)acc[mi][ni][r];
                    out[r] = wide ? dual_rowsum_one<false>(a, r0[0], r0[1], r0[3], r1[1], r1[0], sx, c0[r][0], c0[r][1], s1, s2,
                                                           c0[r][3], c1[r][0], c1[r][1], c1[r][2], BIAS, b)
                                  : dual_rowsum_one<true>(a, r0[0], r0[1], r0[3], r1[1], r1[0], sx, c0[r][0], c0[r][1], s1, s2,
                                                          c0[r][3], c1[r][0], c1[r][1], c1[r][2], BIAS, b);
                }
                *reinterpret_cast<v2u *>(stage + (mi * 16 + l16) * kYStride + ncol * 2) =
                    v2u{(uint32_t)out[0] | ((uint32_t)out[1] << 16), (uint32_t)out[2] | ((uint32_t)out[3] << 16)};
            }
        }
    } else {
#pragma unroll
    for (int ni = 0; ni < TNI; ++ni) {
        const uint32_t ncol = ni * 16 + kb * 4;
        const uint32_t nq = min(n0 + wave * (16 * TNI) + ncol, p.N - 4);
        const QuadCols<MODE, BIAS> cols =
            quad_cols_from_raw<MODE, BIAS>(raw_s1[ni], raw_z1[ni], raw_s2[ni], raw_z2[ni], raw_bias[ni], nq, raw_rs[ni]);
#pragma unroll
        for (int mi = 0; mi < TMI; ++mi) {
            *reinterpret_cast<v2u *>(stage + (mi * 16 + l16) * kYStride + ncol * 2) =
                v2u{dequant_pair<MODE, BIAS>(acc[mi][ni][0], acc[mi][ni][1], rowp[mi], cols.c[0], cols.c[1]),
                    dequant_pair<MODE, BIAS>(acc[mi][ni][2], acc[mi][ni][3], rowp[mi], cols.c[2], cols.c[3])};
        }
    }
    }
    const uint32_t rows_here = min(p.M - m0, (uint32_t)BM);
    const __amdgpu_buffer_rsrc_t rY = make_rsrc(p.y + (uint64_t)m0 * p.N, rows_here * p.N * 2);
    constexpr uint32_t PPR = 2 * TNI, RPI = 64 / PPR;  // 16-byte pieces per staged row, rows per store instruction
    const uint32_t piece = lane % PPR, rsub = lane / PPR;
    const uint32_t ncol0 = n0 + wave * (16 * TNI) + piece * 8;
#pragma unroll
    for (int it = 0; it < BM / (int)RPI; ++it) {
        const uint32_t row = it * RPI + rsub;
        const v4u v = *reinterpret_cast<const v4u *>(stage + row * kYStride + piece * 16);
        const uint32_t off = (row < rows_here && ncol0 < p.N) ? (row * p.N + ncol0) * 2 : kOobOffset;
        __builtin_amdgcn_raw_buffer_store_b128(v, rY, (int)off, 0, DUQ_BF6_STORE_AUX);
    }
}

template <int TMI, int TNI, int EPI>
static void launch_tile(const Bf6Params &p, hipStream_t stream)
{
    const dim3 grid(p.tiles_m * p.tiles_n);
    if (p.epi.bias)
        DUQ_LAUNCH_HEAD((gemm_bf6_kernel<TMI, TNI, EPI, true>), grid, dim3(256), 0, stream, p);
    else
        DUQ_LAUNCH_HEAD((gemm_bf6_kernel<TMI, TNI, EPI, false>), grid, dim3(256), 0, stream, p);
}

template <int EPI>
static void launch_mode(Bf6Params &p, hipStream_t stream)
{
    // Tile height: whole rounds of 256 workgroups, with a 64-row / 256-row tile priced relative to a 128-row one
    // (the weight traffic per tile is the same, the MFMAs are half / twice; measured on an MI355X).
    constexpr float kCost64 = DUQ_BF6_COST64, kCost256 = DUQ_BF6_COST256;
    const uint32_t t256 = ((p.M + 255) / 256) * p.tiles_n, t128 = ((p.M + 127) / 128) * p.tiles_n,
                   t64 = ((p.M + 63) / 64) * p.tiles_n;
    const float c256 = kCost256 * (float)((t256 + 255) / 256), c128 = (float)((t128 + 255) / 256),
                c64 = kCost64 * (float)((t64 + 255) / 256);
    // (the 256-row tile leaves no LDS for the staged parameters of epilogue 5)
    if (EPI != 5 && c256 < c128 && c256 <= c64) {
        p.tiles_m = (p.M + 255) / 256;
        if constexpr (EPI != 5) launch_tile<16, 4, EPI>(p, stream);
    } else if (c64 < c128) {
        p.tiles_m = (p.M + 63) / 64;
        // CUs left without a 64 x 256 tile: 64 x 128 tiles, twice as many, as long as they still run in one round
        // (measured: 23-35 % faster up to 128 tiles of 64 x 256, slower from 160 on)
        if (t64 <= DUQ_BF6_NARROW_MAX_TILES) {
            p.tiles_n = (p.N + 127) / 128;
            launch_tile<4, 2, EPI>(p, stream);
        } else {
            launch_tile<4, 4, EPI>(p, stream);
        }
    } else {
        p.tiles_m = (p.M + 127) / 128;
        launch_tile<8, 4, EPI>(p, stream);
    }
}

int launch_gemm_bf6(const uint8_t *X, const uint8_t *W, uint32_t M, uint32_t N, uint32_t K, const Epilogue &epi,
                    uint16_t *y, hipStream_t stream, const uint8_t *xq, const uint8_t *wq)
{
    if (M == 0 || N == 0) return 0;
    Bf6Params p{X, W, M, N, K, (M + 127) / 128, y, (N + 255) / 256, epi, xq, wq};
    switch (epi.mode) {
    case 0: launch_mode<0>(p, stream); break;
    case 1: launch_mode<1>(p, stream); break;
    case 2: launch_mode<2>(p, stream); break;
    case 3: launch_mode<3>(p, stream); break;
    case 4: launch_mode<4>(p, stream); break;
    case 5:
        if (!xq || !wq) return (int)hipErrorInvalidValue;
        launch_mode<5>(p, stream);
        break;
    default: return (int)hipErrorInvalidValue;
    }
    return (int)hipGetLastError();
}

}  // namespace duq
