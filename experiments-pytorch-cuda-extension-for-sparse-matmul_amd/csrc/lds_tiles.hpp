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
//     alignment survives and 8 consecutive lanes always cover one 128-byte bank
//     window exactly once;
//   * LDS -> MFMA registers is one ds_read_b128 per k-step when the contraction
//     index is contiguous in the tile, and two ds_read_b64_tr_b16 when it is the
//     slow index (the hardware transposes; no shuffles);
//   * tiles belong to ONE wavefront, so no workgroup barrier is involved.
// tests/test_lds_bank_model.py replays every address map below through a model
// of the LDS banks.
#pragma once

#include "bsa_device.hpp"

namespace bsa {

// inverse of perm16
__device__ __forceinline__ int invperm16(int r) { return (r & 3) + 4 * ((r >> 4) & 1) + 8 * ((r >> 2) & 3); }

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

// ---- tile stored [index][k] (contraction contiguous) -----------------------
// LDS slot (16 bytes) of piece p of row r: r * 4 + (p ^ ((r >> 1) & 3)).
__device__ __forceinline__ int kc_slot(int row, int piece) { return row * 4 + (piece ^ ((row >> 1) & 3)); }

// PERMUTED stores global row r at LDS row invperm16(r), so that the reader's
// lane i finds global row perm16(i) at LDS row i.
template <bool PERMUTED>
__device__ __forceinline__ void lds_put_kc(half_t *tile, const uint4 (&raw)[2])
{
    int l = lane_id();
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        int c = l + 64 * q;
        int row = PERMUTED ? invperm16(c >> 2) : (c >> 2);
        *reinterpret_cast<uint4 *>(tile + 8 * kc_slot(row, c & 3)) = raw[q];
    }
}

// halves k = 16 * step + 8 * (lane / 32) + 0..7 of LDS row lane % 32
__device__ __forceinline__ h8 lds_get_kc(const half_t *tile, int step)
{
    int l = lane_id();
    return *reinterpret_cast<const h8 *>(tile + 8 * kc_slot(l & 31, 2 * step + (l >> 5)));
}

// ---- tile stored [k][index] (contraction is the slow index) -----------------
// LDS slot of piece p of row k: k * 4 + (p ^ (2 * ((k >> 1) & 1))): rows k and k + 2
// would otherwise share a bank window for the 32-byte reads of one lane group.
__device__ __forceinline__ int ks_slot(int k, int piece) { return k * 4 + (piece ^ (((k >> 1) & 1) << 1)); }

__device__ __forceinline__ void lds_put_ks(half_t *tile, const uint4 (&raw)[2])
{
    int l = lane_id();
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        int c = l + 64 * q;
        *reinterpret_cast<uint4 *>(tile + 8 * ks_slot(c >> 2, c & 3)) = raw[q];
    }
}

// halves k = 16 * step + 8 * (lane / 32) + 0..7 of index lane % 32 (or perm16 of it)
template <bool PERMUTED>
__device__ __forceinline__ h8 lds_get_ks(const half_t *tile, int step)
{
    int l = lane_id();
    int g = l >> 4, s = l & 15;
    int k = 16 * step + 8 * (g >> 1) + (s >> 2);
    int x = tr_chunk_base<PERMUTED>(g, s & 3) ^ (((k >> 1) & 1) << 4);   // k + 4 swizzles alike
    h4 lo = lds_read_tr16(tile + k * BS + x);
    h4 hi = lds_read_tr16(tile + (k + 4) * BS + x);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// ---- result tile: 32 rows x 32 halves, lane (row = lane % 32, h = lane / 32)
// holds columns 16 h .. 16 h + 15; written swizzled, read back in tile order so
// the global store is the same coalesced request as the loads.
__device__ __forceinline__ void lds_put_result(half_t *tile, const uint4 &lo, const uint4 &hi)
{
    int l = lane_id();
    int row = l & 31, p = 2 * (l >> 5);
    *reinterpret_cast<uint4 *>(tile + 8 * kc_slot(row, p)) = lo;
    *reinterpret_cast<uint4 *>(tile + 8 * kc_slot(row, p + 1)) = hi;
}

__device__ __forceinline__ void lds_get_linear(const half_t *tile, uint4 (&raw)[2])
{
    int l = lane_id();
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        int c = l + 64 * q;
        raw[q] = *reinterpret_cast<const uint4 *>(tile + 8 * kc_slot(c >> 2, c & 3));
    }
}

// coalesced store of a 2 KB block
__device__ __forceinline__ void stg_tile32(half_t *dst, const uint4 (&raw)[2])
{
    int l = lane_id();
    stg16(dst + 8 * l, raw[0]);
    stg16(dst + 8 * (l + 64), raw[1]);
}

}  // namespace bsa
