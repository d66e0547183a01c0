// Helpers shared by the GEMM kernels: workgroup -> tile mapping for the eight XCDs and raw
// buffer descriptors (out-of-range reads return zero without a branch).
#pragma once
#include "duq_device.h"

namespace duq {

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

constexpr uint32_t kOobOffset = 0xFFFFFF00u;  // beyond any descriptor: the load returns 0

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ v4u buf_load16(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff)
{
    return __builtin_bit_cast(v4u, __builtin_amdgcn_raw_buffer_load_b128(r, (int)voff, (int)soff, 0));
}
// The same with a cache policy (2 = non-temporal: for bytes that are read once, in whole cache lines).
template <int AUX>
__device__ __forceinline__ v4u buf_load16_aux(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff)
{
    return __builtin_bit_cast(v4u, __builtin_amdgcn_raw_buffer_load_b128(r, (int)voff, (int)soff, AUX));
}

}  // namespace duq
