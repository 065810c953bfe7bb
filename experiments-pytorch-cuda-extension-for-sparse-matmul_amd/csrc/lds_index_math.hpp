// Pure index arithmetic of the LDS tile layouts and of the MFMA lane maps, usable
// on the host and on the device.  Kept free of HIP so that the same functions the
// kernels use can be compiled with g++ and replayed through the LDS bank model
// (tests/test_lds_bank_model.py).  Units: a "piece" is 16 bytes = 8 halves.
#pragma once

#if defined(__HIPCC__)
#define BSA_HD __host__ __device__ __forceinline__
#else
#define BSA_HD inline
#endif

namespace bsa {

// MFMA 32x32 accumulators give lane (l % 32, h = l / 32) the result rows
// 8 * (v / 4) + 4 * h + v % 4, v = 0..15.  Feeding the row operand through this
// permutation makes those 16 values 16 CONSECUTIVE logical indices 16 * h + v,
// so a lane can store them with two 16-byte (fp16) or four (fp32) writes.
BSA_HD constexpr int perm16(int i) { return (i & 3) + 4 * (i >> 3) + 16 * ((i >> 2) & 1); }
BSA_HD constexpr int invperm16(int r) { return (r & 3) + 4 * ((r >> 4) & 1) + 8 * ((r >> 2) & 3); }

// Tile stored [index][k] (contraction contiguous), 64-byte rows: 16-byte slot of
// piece p of row r.  An operand read takes the SAME piece of 16 consecutive rows
// per 16-lane phase; rows r, r + 4, r + 8, r + 12 start at the same offset of the
// 256-byte bank window, so the XOR sends them to the four different pieces.  The
// mask depends on r % 16 only: lanes i and i + 16 of a 32-lane half must use the
// same banks or the read takes twice as long (measured with lds_bank_probe).
BSA_HD constexpr int kc_swizzle(int row) { return (row >> 2) & 3; }
BSA_HD constexpr int kc_slot(int row, int piece) { return row * 4 + (piece ^ kc_swizzle(row)); }

// Tile stored [k][index] (contraction is the slow index), 64-byte rows.  A lane
// group of a transposing read takes two pieces ({0,1}, {2,3}, {0,2} or {1,3}) of 4
// consecutive rows; rows k and k + 2 share a bank window and flip both piece bits.
BSA_HD constexpr int ks_swizzle(int k) { return 3 * ((k >> 1) & 1); }
BSA_HD constexpr int ks_slot(int k, int piece) { return k * 4 + (piece ^ ks_swizzle(k)); }

// [k][64] dense strip, 128-byte rows (8 pieces): a lane group takes pieces
// {2m, 2m+1} or {j, j+2} of 4 consecutive rows; the four XOR masks 0, 3, 4, 7 keep
// both kinds of pairs apart across the rows.
BSA_HD constexpr int strip_swizzle(int k) { return 3 * (k & 1) + 4 * ((k >> 1) & 1); }

// Column (in halves) that source-lane quad a of lane group g = lane / 16 hands to
// ds_read_b64_tr_b16 so that result lane l ends up with index l % 32 (natural) or
// perm16(l % 32) (permuted).
BSA_HD constexpr int tr_chunk_base(bool permuted, int g, int a)
{
    return permuted ? 8 * (g & 1) + 4 * (a >> 1) + 16 * (a & 1) : 16 * (g & 1) + 4 * a;
}

// ---- byte addresses inside a wave-private tile, per lane ---------------------

// registers -> LDS of a [index][k] tile: piece c = lane + 64 q of the 2 KB tile
BSA_HD constexpr int put_kc_addr(bool permuted, int lane, int q)
{
    int c = lane + 64 * q;
    int row = permuted ? invperm16(c >> 2) : (c >> 2);
    return 16 * kc_slot(row, c & 3);
}
// LDS -> MFMA operand, k-step `step`
BSA_HD constexpr int get_kc_addr(int lane, int step) { return 16 * kc_slot(lane & 31, 2 * step + (lane >> 5)); }

BSA_HD constexpr int put_ks_addr(int lane, int q)
{
    int c = lane + 64 * q;
    return 16 * ks_slot(c >> 2, c & 3);
}
// address handed to ds_read_b64_tr_b16 (8 bytes per lane); half = 0 for k..k+3, 1 for k+4..k+7
BSA_HD constexpr int get_ks_addr(bool permuted, int lane, int step, int half)
{
    int g = lane >> 4, s = lane & 15;
    int k = 16 * step + 8 * (g >> 1) + (s >> 2) + 4 * half;
    int x = tr_chunk_base(permuted, g, s & 3) ^ (8 * ks_swizzle(k));   // k + 4 swizzles alike
    return 2 * (k * 32 + x);
}

// [k][64] dense strip (group walk, contraction slow): piece c = lane + 64 q of the 4 KB strip
BSA_HD constexpr int put_strip_addr(int lane, int q)
{
    int c = lane + 64 * q;
    int k = c >> 3;
    return 16 * (k * 8 + ((c & 7) ^ strip_swizzle(k)));
}
// The same strip with rows 4-7 and 8-11 of every 16 exchanged (bits 2 and 3 of k): a reader
// that asks for row 16 s + 8 h + j then gets row 16 s + 8 (j / 4) + 4 h + j % 4, the row an MFMA
// accumulator lane (h = lane / 32) holds as its value 8 s + j.  The fused attention kernel feeds its
// probabilities to the second product straight out of the first one's accumulators this way.
BSA_HD constexpr int swap_bits23(int k) { return (k & ~12) | ((k & 4) << 1) | ((k & 8) >> 1); }
BSA_HD constexpr int put_strip_swapped_addr(int lane, int q)
{
    int c = lane + 64 * q;
    int k = swap_bits23(c >> 3);
    return 16 * (k * 8 + ((c & 7) ^ strip_swizzle(k)));
}
// Transposing read of a [index][k] tile (the put_kc_addr layout, not permuted) along its ROWS: the
// operand of a product that contracts over the tile's row index, with the same exchange of rows
// 4-7 and 8-11 as above applied by the reader: element j of lane (index = lane % 32, h = lane / 32)
// is row 16 step + 8 (j / 4) + 4 h + j % 4.  The 4 rows a 16-lane group touches share one
// kc_swizzle and fill one 256-byte bank window.
BSA_HD constexpr int get_kc_tr_swapped_addr(int lane, int step, int half)
{
    int g = lane >> 4, s = lane & 15;
    int k = 16 * step + 4 * (g >> 1) + (s >> 2) + 8 * half;
    int x = tr_chunk_base(false, g, s & 3) ^ (8 * kc_swizzle(k));
    return 2 * (k * 32 + x);
}
BSA_HD constexpr int get_strip_addr(bool permuted, int lane, int step, int half, int x0)
{
    int g = lane >> 4, s = lane & 15;
    int k = 16 * step + 8 * (g >> 1) + (s >> 2) + 4 * half;   // k + 4 swizzles alike
    int x = (x0 + tr_chunk_base(permuted, g, s & 3)) ^ (8 * strip_swizzle(k));
    return 2 * (k * 64 + x);
}

// ---- the same [k][64] strip as the row operand of v_mfma_f32_16x16x32 (16 columns x 32 k per product) ----
// Lane (g = lane / 16, i = lane % 16) of that operand holds k = 8 g .. 8 g + 7 of ONE column, and the
// accumulator of lane (g, .) holds rows 4 g + v.  Product t (0..3) of a block takes the columns
//   col16(t, i) = 8 (i / 4) + 32 (t / 2) + 4 (t % 2) + i % 4,
// so that accumulators t = 0, 1 of a lane are 8 consecutive columns 8 g .. 8 g + 7 and t = 2, 3 the
// same 32 further on: two 16-byte stores per lane and output row.  A 32-lane phase of the transposing
// read holds two 16-lane groups whose rows are 8 apart and swizzle alike, each touching one 8-byte
// half of 16 pieces; rows 8-15 and 24-31 are therefore stored with the two halves of every piece
// exchanged (bit 3 of k), which sends the two groups to complementary banks.
BSA_HD constexpr int col16(int t, int i) { return 8 * (i >> 2) + 32 * (t >> 1) + 4 * (t & 1) + (i & 3); }
BSA_HD constexpr int strip16_half_swapped(int k) { return (k >> 3) & 1; }
// registers -> LDS: piece c = lane + 64 q as in put_strip_addr; the caller exchanges the halves of
// the piece when strip16_half_swapped(row) (the row is 8 q + lane / 8, so that is q & 1)
BSA_HD constexpr int put_strip16_addr(int lane, int q) { return put_strip_addr(lane, q); }
// address handed to ds_read_b64_tr_b16 for product t; half = 0 for k .. k + 3, 1 for k + 4 .. k + 7
BSA_HD constexpr int get_strip16_addr(int lane, int t, int half)
{
    int g = lane >> 4, s = lane & 15;
    int k = 8 * g + 4 * half + (s >> 2);
    int piece = ((s & 3) + 4 * (t >> 1)) ^ strip_swizzle(k);
    int hp = (t & 1) ^ strip16_half_swapped(k);
    return 128 * k + 16 * piece + 8 * hp;
}

// result tile (SDD): lane (row = lane % 32, h = lane / 32) parks columns 16 h .. 16 h + 15
BSA_HD constexpr int put_result_addr(int lane, int j) { return 16 * kc_slot(lane & 31, 2 * (lane >> 5) + j); }
BSA_HD constexpr int get_linear_addr(int lane, int q)
{
    int c = lane + 64 * q;
    return 16 * kc_slot(c >> 2, c & 3);
}

// ---- fp32 tiles (32 x 32 floats = 4 KB, stored in their memory orientation) ---------------------
// Row r of the tile starts 36 r floats into the LDS tile, rows 16-31 another 32 floats on.  A 16-lane
// phase of a 16-byte access that takes the same columns of 16 different rows then touches 16 different
// groups of four banks (9 r + 8 [r >= 16] mod 16 runs through all of them for r = 0..15, for 16..31 and
// for both halves of the perm16 order), and a 4-byte access of 32 consecutive columns of row k by the
// lower lane half and of row k + 16 by the upper half covers all 64 banks once.  The linear access
// (put_f32_addr: a phase takes the 8 pieces of two NEIGHBOURING rows, whose 32-float windows are 36
// floats apart) meets in 4 of the 64 banks: two clocks per phase instead of one.  Phases that take rows
// 16 apart are conflict-free, but their requests cover a stored block in two runs of 512 bytes instead
// of one kilobyte, and the group walks measured 2-4 us slower with them at 4096 tokens, 16 heads.
constexpr int F32_TILE_FLOATS = 32 * 36 + 32;
BSA_HD constexpr int f32_tile_off(int row, int col) { return row * 36 + ((row >> 4) << 5) + col; }
// registers <-> LDS in memory order, 16 bytes per lane: request j of lane l moves piece
// (row l / 8 + 8 j, columns 4 (l % 8) .. + 3); the 64 lanes of a request cover 8 whole consecutive rows
BSA_HD constexpr int put_f32_addr(int lane, int j) { return 4 * f32_tile_off((lane >> 3) + 8 * j, 4 * (lane & 7)); }
// LDS -> MFMA operand (v_mfma_f32_32x32x2_f32: lane = index, k = 16 (lane / 32) + 0..15), tile stored
// [index][k]: 16-byte read q gives k = 16 h + 4 q .. + 3.  The SDD result (lane = row, 16 consecutive
// columns 16 h ..) is parked with the same addresses.
BSA_HD constexpr int get_f32_kc_addr(bool permuted, int lane, int q)
{
    return 4 * f32_tile_off(permuted ? perm16(lane & 31) : (lane & 31), 16 * (lane >> 5) + 4 * q);
}
// tile stored [k][index]: 4-byte read t gives k = 16 h + t
BSA_HD constexpr int get_f32_ks_addr(bool permuted, int lane, int t)
{
    return 4 * f32_tile_off(16 * (lane >> 5) + t, permuted ? perm16(lane & 31) : (lane & 31));
}

}  // namespace bsa
