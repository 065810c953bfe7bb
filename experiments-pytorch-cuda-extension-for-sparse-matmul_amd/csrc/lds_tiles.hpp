// Wave-private LDS staging of 32 x 32 fp16 operand tiles.
//
// This is the gfx950 counterpart of the reference's tile<T, ROWS, COLS>
// storage / loader pair (native/tiling_utils.cuh:12-98: a padded, double-buffered
// shared-memory tile filled 4 bytes per thread, with a warp-shuffle transpose for
// fp16).  Here:
//   * global -> registers is always the same fully coalesced request: lane l
//     fetches the 16-byte pieces l and l + 64 of the 2 KB tile (4 pieces = one
//     64-byte row), whatever the orientation of the operand;
//   * registers -> LDS applies an XOR swizzle instead of padding, so 16-byte
//     alignment survives and every access is free of bank conflicts for a
//     32-bank as well as for a 64-bank LDS;
//   * LDS -> MFMA registers is one ds_read_b128 per k-step when the contraction
//     index is contiguous in the tile, and two ds_read_b64_tr_b16 when it is the
//     slow index (the hardware transposes; no shuffles);
//   * tiles belong to ONE wavefront, so no workgroup barrier is involved.
// tests/test_lds_bank_model.py replays every address map below through a model
// of the LDS banks.
#pragma once

#include "bsa_device.hpp"

namespace bsa {

// Coalesced load of a 32 x 32 half tile whose rows are `ld` halves apart.
__device__ __forceinline__ void ldg_tile32(const half_t *src, size_t ld, uint4 (&raw)[2])
{
    int l = lane_id();
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        int c = l + 64 * q;
        raw[q] = ldg16(src + (size_t)(c >> 2) * ld + 8 * (c & 3));
    }
}

// Every LDS byte address below comes from lds_index_math.hpp, the same functions the
// host-side bank-model test replays.
__device__ __forceinline__ unsigned char *lds_bytes(half_t *t) { return reinterpret_cast<unsigned char *>(t); }
__device__ __forceinline__ const unsigned char *lds_bytes(const half_t *t) { return reinterpret_cast<const unsigned char *>(t); }

// ---- tile stored [index][k] (contraction contiguous) -----------------------
// PERMUTED stores global row r at LDS row invperm16(r), so that the reader's
// lane i finds global row perm16(i) at LDS row i.
template <bool PERMUTED>
__device__ __forceinline__ void lds_put_kc(half_t *tile, const uint4 (&raw)[2])
{
    int l = lane_id();
#pragma unroll
    for (int q = 0; q < 2; ++q)
        *reinterpret_cast<uint4 *>(lds_bytes(tile) + put_kc_addr(PERMUTED, l, q)) = raw[q];
}

// halves k = 16 * step + 8 * (lane / 32) + 0..7 of LDS row lane % 32
__device__ __forceinline__ h8 lds_get_kc(const half_t *tile, int step)
{
    return *reinterpret_cast<const h8 *>(lds_bytes(tile) + get_kc_addr(lane_id(), step));
}

// ---- tile stored [k][index] (contraction is the slow index) -----------------
__device__ __forceinline__ void lds_put_ks(half_t *tile, const uint4 (&raw)[2])
{
    int l = lane_id();
#pragma unroll
    for (int q = 0; q < 2; ++q)
        *reinterpret_cast<uint4 *>(lds_bytes(tile) + put_ks_addr(l, q)) = raw[q];
}

// halves k = 16 * step + 8 * (lane / 32) + 0..7 of index lane % 32 (or perm16 of it)
template <bool PERMUTED>
__device__ __forceinline__ h8 lds_get_ks(const half_t *tile, int step)
{
    int l = lane_id();
    h4 lo = lds_read_tr16(reinterpret_cast<const half_t *>(lds_bytes(tile) + get_ks_addr(PERMUTED, l, step, 0)));
    h4 hi = lds_read_tr16(reinterpret_cast<const half_t *>(lds_bytes(tile) + get_ks_addr(PERMUTED, l, step, 1)));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// rows of a [index][k] tile as the contraction, rows 4-7 and 8-11 of every 16 exchanged (see get_kc_tr_swapped_addr)
__device__ __forceinline__ h8 lds_get_kc_tr_swapped(const half_t *tile, int step)
{
    int l = lane_id();
    h4 lo = lds_read_tr16(reinterpret_cast<const half_t *>(lds_bytes(tile) + get_kc_tr_swapped_addr(l, step, 0)));
    h4 hi = lds_read_tr16(reinterpret_cast<const half_t *>(lds_bytes(tile) + get_kc_tr_swapped_addr(l, step, 1)));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// ---- [k][64] dense strip, 128-byte rows, XOR swizzle (group walk) -------------
__device__ __forceinline__ void lds_put_strip(half_t *tile, const uint4 (&lo)[2], const uint4 (&hi)[2])
{
    int l = lane_id();
#pragma unroll
    for (int q = 0; q < 4; ++q)
        *reinterpret_cast<uint4 *>(lds_bytes(tile) + put_strip_addr(l, q)) = q < 2 ? lo[q & 1] : hi[q & 1];
}

// rows 4-7 and 8-11 of every 16 exchanged (see put_strip_swapped_addr)
__device__ __forceinline__ void lds_put_strip_swapped(half_t *tile, const uint4 (&raw)[4])
{
    int l = lane_id();
#pragma unroll
    for (int q = 0; q < 4; ++q)
        *reinterpret_cast<uint4 *>(lds_bytes(tile) + put_strip_swapped_addr(l, q)) = raw[q];
}

template <bool PERMUTED>
__device__ __forceinline__ h8 lds_get_strip(const half_t *tile, int x0, int step)
{
    int l = lane_id();
    h4 lo = lds_read_tr16(reinterpret_cast<const half_t *>(lds_bytes(tile) + get_strip_addr(PERMUTED, l, step, 0, x0)));
    h4 hi = lds_read_tr16(reinterpret_cast<const half_t *>(lds_bytes(tile) + get_strip_addr(PERMUTED, l, step, 1, x0)));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// ---- result tile: 32 rows x 32 halves, lane (row = lane % 32, h = lane / 32)
// holds columns 16 h .. 16 h + 15; written swizzled, read back in tile order so
// the global store is the same coalesced request as the loads.
__device__ __forceinline__ void lds_put_result(half_t *tile, const uint4 &lo, const uint4 &hi)
{
    int l = lane_id();
    *reinterpret_cast<uint4 *>(lds_bytes(tile) + put_result_addr(l, 0)) = lo;
    *reinterpret_cast<uint4 *>(lds_bytes(tile) + put_result_addr(l, 1)) = hi;
}

__device__ __forceinline__ void lds_get_linear(const half_t *tile, uint4 (&raw)[2])
{
    int l = lane_id();
#pragma unroll
    for (int q = 0; q < 2; ++q)
        raw[q] = *reinterpret_cast<const uint4 *>(lds_bytes(tile) + get_linear_addr(l, q));
}

// coalesced store of a 2 KB block (written once, not read again by this kernel)
__device__ __forceinline__ void stg_tile32(half_t *dst, const uint4 (&raw)[2])
{
    int l = lane_id();
    stg16_stream(dst + 8 * l, raw[0]);
    stg16_stream(dst + 8 * (l + 64), raw[1]);
}

// coalesced load of a contiguous 2 KB block that is read once
__device__ __forceinline__ void ldg_block32_stream(const half_t *src, uint4 (&raw)[2])
{
    int l = lane_id();
    raw[0] = ldg16_stream(src + 8 * l);
    raw[1] = ldg16_stream(src + 8 * (l + 64));
}

}  // namespace bsa
