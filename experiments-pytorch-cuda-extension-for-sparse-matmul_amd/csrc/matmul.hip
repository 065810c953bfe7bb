// SDD / DSD / DDS block-sparse matmul for gfx950.
//
// Replaces the three kernels of sparse/native/sparse_smm_gpu.cu:22-267 and the
// unfinished fp16 twin sparse/native/sparse_hmm_gpu.cu:26-317.  Nothing of
// their structure is kept: every nonzero 32x32 block is one MFMA tile owned by
// ONE wavefront (v_mfma_f32_32x32x16_f16, fp32 accumulate; v_mfma_f32_32x32x2_f32
// for fp32).  Tiles are fetched with fully coalesced requests (lane l takes
// 16-byte pieces l and l + 64 of a 2 KB fp16 tile, whatever its orientation; a
// request of an fp32 tile covers 8 whole 128-byte rows), parked in a wave-private
// LDS tile (XOR-swizzled for fp16, padded rows for fp32) and read back in MFMA
// layout: ds_read_b128 when the contraction index is contiguous in the tile,
// ds_read_b64_tr_b16 (hardware transpose; ds_read_b32 for fp32) when it is the
// slow index.  MFMA-layout loads straight from global memory (lane = row, 16
// bytes at row stride) were measured at a third of the coalesced rate; only the
// fp32 fallbacks (K > 128, a dense dimension that is no multiple of 64) keep
// them.  Data touched once (sparse blocks, results) moves with non-temporal
// loads and stores; dense tiles, which are re-read out of L2, do not.  No
// workgroup barrier sits in any inner loop, and no load under a condition sits
// in the steady state of a block loop (tails are peeled): behind a conditional
// load the compiler can no longer count the loads in flight and waits for all of
// them, which cancels the prefetch.
//
// Work distribution: a schedule (see bsa.h) hands every wavefront a chunk of
// consecutive table pairs of one group.  SDD: the chunk's blocks share the
// block row, whose dense rows are kept in registers.  DSD/DDS ("group walk"):
// the waves of a team accumulate partial 32x64 tiles and reduce through LDS.
//
// MFMA roles.  Of the two operands the one indexed by the accumulator REGISTER
// (v) is fed through perm16 so a lane ends up with 16 consecutive output
// elements; it is always the operand that runs along the contiguous dimension
// of the output.  The other operand is indexed by the lane.
#include <mutex>

#include "bsa_device.hpp"
#include "lds_tiles.hpp"
#include "bsa_internal.hpp"
#include "group_walk.hpp"
#include "../../include/bsa.h"

namespace bsa {

#ifndef BSA_GW_DEPTH
#define BSA_GW_DEPTH 2
#endif
constexpr int GW_PREFETCH_DEPTH = BSA_GW_DEPTH;    // pairs whose operands are in flight per wave: deeper costs 24 VGPRs a
                                        // stage and did not pay (124 VGPRs = 4 waves per SIMD at depth 2)
constexpr int SDD_KB_MAX = 4;           // k-blocks (of 32) whose operands stay resident per wave
constexpr int SDD_LDS_PER_WAVE = 2048 * (1 + SDD_KB_MAX);   // a / result tile + one b tile per k-block

// ---------------------------------------------------------------------------
// SDD fp16
// ---------------------------------------------------------------------------
template <bool A_KC, bool B_KC, int KBT, bool BF>
__global__ __launch_bounds__(512) void sdd_f16_kernel(
    const half_t *__restrict__ a, const half_t *__restrict__ b, half_t *__restrict__ c,
    const BlockDesc *__restrict__ blocks, const SchedEntry *__restrict__ sched,
    int n_swg, int batches, int nnz, int M, int N, int K)
{
    extern __shared__ __align__(16) unsigned char lds_raw[];
    int batch, swg;
    if (!map_workgroup(n_swg, batches, batch, swg)) return;
    const int w = wave_id();
    const int W = (int)(blockDim.x >> 6);
    const SchedEntry e = sched[swg * W + w];
    if (e.group < 0 || e.begin >= e.end) return;

    half_t *tile_a = reinterpret_cast<half_t *>(lds_raw + (size_t)w * SDD_LDS_PER_WAVE);
    half_t *tile_c = tile_a;            // the a tile is dead once its operands sit in registers
    half_t *tile_b = tile_a + BS2;      // KBT (or 1) tiles
    const half_t *ab = a + (size_t)batch * M * K;
    const half_t *bb = b + (size_t)batch * N * K;
    half_t *cb = c + (size_t)batch * nnz * BS2;
    const int r = e.group;

    // op(a) rows of the block row: [M][K] storage is contraction-contiguous, [K][M] is not
    auto load_a = [&](int kb, uint4(&raw)[2]) {
        if (A_KC) ldg_tile32(ab + (size_t)(BS * r) * K + BS * kb, K, raw);
        else ldg_tile32(ab + (size_t)(BS * kb) * M + BS * r, M, raw);
    };
    // op(b) columns of the block column: [N][K] storage is contraction-contiguous, [K][N] is not
    auto load_b = [&](int cblk, int kb, uint4(&raw)[2]) {
        if (B_KC) ldg_tile32(bb + (size_t)(BS * cblk) * K + BS * kb, K, raw);
        else ldg_tile32(bb + (size_t)(BS * kb) * N + BS * cblk, N, raw);
    };
    auto put_a = [&](half_t *t, const uint4(&raw)[2]) { if (A_KC) lds_put_kc<false>(t, raw); else lds_put_ks(t, raw); };
    auto put_b = [&](half_t *t, const uint4(&raw)[2]) { if (B_KC) lds_put_kc<true>(t, raw); else lds_put_ks(t, raw); };
    auto get_a = [&](const half_t *t, int s) { return A_KC ? lds_get_kc(t, s) : lds_get_ks<false>(t, s); };
    auto get_b = [&](const half_t *t, int s) { return B_KC ? lds_get_kc(t, s) : lds_get_ks<true>(t, s); };
    // the b operand feeds the accumulator-register index (through perm16), so a lane ends up
    // with 16 consecutive columns of its row; the block leaves through LDS as whole 2 KB
    auto store = [&](int idx, const f16v &acc) {
        uint4 lo, hi, raw[2];
        pack16<BF>(acc, lo, hi);
        wave_lds_fence();
        lds_put_result(tile_c, lo, hi);
        wave_lds_fence();
        lds_get_linear(tile_c, raw);
        stg_tile32(cb + (size_t)idx * BS2, raw);
    };

    if (KBT > 0) {
        constexpr int KB = KBT > 0 ? KBT : 1;
        // The wave's first requests all go out together: its block descriptors, the A tiles of every
        // k-block, then (as soon as the descriptors are back) the B tiles of its first block; the A tiles
        // are turned into operand registers while those are in flight.  One memory round trip instead
        // of one per k-block plus one for the descriptors plus one for the first block.
        h8 aop[KB][2];
        uint4 araw[KB][2], braw[2][KB][2];
        DescWindow win;
        const int first_end = e.begin + WAVE < e.end ? e.begin + WAVE : e.end;
        win.fetch(blocks, e.begin, first_end);
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) load_a(kb, araw[kb]);
        auto load_tiles = [&](int p, uint4 (&raw)[KB][2]) {
            const int cblk = win.get(p).col();
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) load_b(cblk, kb, raw[kb]);
        };
        auto multiply = [&](int p, const uint4 (&raw)[KB][2]) {
            wave_lds_fence();
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) put_b(tile_b + kb * BS2, raw[kb]);
            wave_lds_fence();
            h8 bop[KB][2];
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                bop[kb][0] = get_b(tile_b + kb * BS2, 0);
                bop[kb][1] = get_b(tile_b + kb * BS2, 1);
            }
            f16v acc = {0};
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                acc = mfma_16<BF>(bop[kb][0], aop[kb][0], acc);
                acc = mfma_16<BF>(bop[kb][1], aop[kb][1], acc);
            }
            store(win.get(p).idx, acc);
        };
        // One block ahead: the tiles of block p + 1 are requested before block p is multiplied.  A load
        // under a condition makes the compiler wait for every load and store in flight before the next
        // use, which would cancel the prefetch, so the loop body holds none; the last one or two blocks
        // of a segment are straight-line code.
        load_tiles(e.begin, braw[0]);
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
            wave_lds_fence();
            put_a(tile_a, araw[kb]);
            wave_lds_fence();
            aop[kb][0] = get_a(tile_a, 0);
            aop[kb][1] = get_a(tile_a, 1);
        }
        for (int seg = e.begin; seg < e.end; seg += WAVE) {
            const int seg_end = seg + WAVE < e.end ? seg + WAVE : e.end;
            if (seg != e.begin) {
                win.fetch(blocks, seg, seg_end);
                load_tiles(seg, braw[0]);
            }
            int p = seg;
            for (; p + 2 < seg_end; p += 2) {
                load_tiles(p + 1, braw[1]);
                multiply(p, braw[0]);
                load_tiles(p + 2, braw[0]);
                multiply(p + 1, braw[1]);
            }
            if (p + 1 < seg_end) {
                load_tiles(p + 1, braw[1]);
                multiply(p, braw[0]);
                multiply(p + 1, braw[1]);
            } else {
                multiply(p, braw[0]);
            }
        }
    } else {
        const int kbs = K / BS;
        DescWindow win;
        for (int p = e.begin; p < e.end; ++p) {
            if (((p - e.begin) & (WAVE - 1)) == 0) win.fetch(blocks, p, e.end);
            const BlockDesc d = win.get(p);
            f16v acc = {0};
            uint4 araw[2], braw[2];
            load_a(0, araw);
            load_b(d.col(), 0, braw);
            for (int kb = 0; kb < kbs; ++kb) {
                wave_lds_fence();
                put_a(tile_a, araw);
                put_b(tile_b, braw);
                wave_lds_fence();
                if (kb + 1 < kbs) {
                    load_a(kb + 1, araw);
                    load_b(d.col(), kb + 1, braw);
                }
                acc = mfma_16<BF>(get_b(tile_b, 0), get_a(tile_a, 0), acc);
                acc = mfma_16<BF>(get_b(tile_b, 1), get_a(tile_a, 1), acc);
            }
            store(d.idx, acc);
        }
    }
}

// ---------------------------------------------------------------------------
// fp32 operand tiles: 16 floats per lane, k = 16 * (lane / 32) + 0..15 of one
// index.  Both memory orientations load straight into registers (the fallback
// kernels sdd_f32_kernel and gw_f32_kernel; the tiled kernels below stage through LDS).
// ---------------------------------------------------------------------------
template <bool KC, bool PERMUTED>
__device__ __forceinline__ void ldg_tile_f32(const float *src, size_t ld, float (&v)[16])
{
    int l = lane_id();
    int i = PERMUTED ? perm16(l & 31) : (l & 31);
    int k0 = 16 * (l >> 5);
    if (KC) {   // src -> [index 0][k 0]
        const float4 *p = reinterpret_cast<const float4 *>(src + (size_t)i * ld + k0);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            float4 x = p[t];
            v[4 * t] = x.x; v[4 * t + 1] = x.y; v[4 * t + 2] = x.z; v[4 * t + 3] = x.w;
        }
    } else {    // src -> [k 0][index 0]
#pragma unroll
        for (int t = 0; t < 16; ++t) v[t] = src[(size_t)(k0 + t) * ld + i];
    }
}

__device__ __forceinline__ void store16_f32(float *o, const f16v &acc)
{
#pragma unroll
    for (int t = 0; t < 4; ++t)
        *reinterpret_cast<float4 *>(o + 4 * t) =
            make_float4(acc[4 * t], acc[4 * t + 1], acc[4 * t + 2], acc[4 * t + 3]);
}

template <bool A_KC, bool B_KC>
__global__ __launch_bounds__(512) void sdd_f32_kernel(
    const float *__restrict__ a, const float *__restrict__ b, float *__restrict__ c,
    const BlockDesc *__restrict__ blocks, const SchedEntry *__restrict__ sched,
    int n_swg, int batches, int nnz, int M, int N, int K)
{
    int batch, swg;
    if (!map_workgroup(n_swg, batches, batch, swg)) return;
    const int w = wave_id(), l = lane_id();
    const int W = (int)(blockDim.x >> 6);
    const SchedEntry e = sched[swg * W + w];
    if (e.group < 0 || e.begin >= e.end) return;
    const float *ab = a + (size_t)batch * M * K;
    const float *bb = b + (size_t)batch * N * K;
    float *cb = c + (size_t)batch * nnz * BS2;
    const int r = e.group, kbs = K / BS;

    DescWindow win;
    for (int p = e.begin; p < e.end; ++p) {
        if (((p - e.begin) & (WAVE - 1)) == 0) win.fetch(blocks, p, e.end);
        const BlockDesc d = win.get(p);
        const int cblk = d.col();
        f16v acc = {0};
        auto load = [&](int kb, float (&av)[16], float (&bv)[16]) {
            if (A_KC) ldg_tile_f32<true, false>(ab + (size_t)(BS * r) * K + BS * kb, K, av);
            else ldg_tile_f32<false, false>(ab + (size_t)(BS * kb) * M + BS * r, M, av);
            if (B_KC) ldg_tile_f32<true, true>(bb + (size_t)(BS * cblk) * K + BS * kb, K, bv);
            else ldg_tile_f32<false, true>(bb + (size_t)(BS * kb) * N + BS * cblk, N, bv);
        };
        // two k-blocks per round: both sets of loads are in flight before the first product
        for (int kb = 0; kb < kbs; kb += 2) {
            float av0[16], bv0[16], av1[16], bv1[16];
            const bool two = kb + 1 < kbs;
            load(kb, av0, bv0);
            if (two) load(kb + 1, av1, bv1);
#pragma unroll
            for (int t = 0; t < 16; ++t) acc = mfma_f32(bv0[t], av0[t], acc);
            if (two) {
#pragma unroll
                for (int t = 0; t < 16; ++t) acc = mfma_f32(bv1[t], av1[t], acc);
            }
        }
        store16_f32(cb + (size_t)d.idx * BS2 + (l & 31) * BS + 16 * (l >> 5), acc);
    }
}

// ---------------------------------------------------------------------------
// fp32 operand tiles through LDS.  A 32 x 32 fp32 tile (rows 128 bytes) is fetched with four fully
// coalesced requests (a request covers 8 whole rows) and parked in a wave-private LDS tile in its memory
// orientation, rows padded: the address maps put_f32_addr / get_f32_kc_addr / get_f32_ks_addr of
// lds_index_math.hpp (byte addresses; the bank-model tests replay them).  The MFMA
// operand (16 floats per lane: one index, k = 16 (lane / 32) .. + 15) is read back with four
// ds_read_b128 when k is the contiguous index and with sixteen ds_read_b32 when k is the row.
// ---------------------------------------------------------------------------
constexpr int F32_TILE_BYTES = 4864;     // F32_TILE_FLOATS floats, rounded up to 128 bytes
static_assert(4 * F32_TILE_FLOATS <= F32_TILE_BYTES, "fp32 tile size");
template <bool STREAM>
__device__ __forceinline__ void ldg_tile32_f32(const float *src, size_t ld, uint4 (&raw)[4])
{
    const int l = lane_id();
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float *p = src + (size_t)((l >> 3) + 8 * j) * ld + 4 * (l & 7);
        raw[j] = STREAM ? ldg16_stream(p) : ldg16(p);
    }
}

__device__ __forceinline__ void lds_put_f32(float *tile, const uint4 (&raw)[4])
{
    const int l = lane_id();
#pragma unroll
    for (int j = 0; j < 4; ++j)
        *reinterpret_cast<uint4 *>(tile + put_f32_addr(l, j) / 4) = raw[j];
}

template <bool KC, bool PERMUTED>
__device__ __forceinline__ void lds_get_f32(const float *tile, float (&v)[16])
{
    const int l = lane_id();
    if (KC) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float4 x = *reinterpret_cast<const float4 *>(tile + get_f32_kc_addr(PERMUTED, l, q) / 4);
            v[4 * q] = x.x; v[4 * q + 1] = x.y; v[4 * q + 2] = x.z; v[4 * q + 3] = x.w;
        }
    } else {
#pragma unroll
        for (int t = 0; t < 16; ++t) v[t] = tile[get_f32_ks_addr(PERMUTED, l, t) / 4];
    }
}

// SDD fp32 with K = 32 KBT <= 128: the operands of the wave's block row stay in registers (16 KBT floats per
// lane), the tiles of block p + 1 are requested as soon as those of block p have left their registers for LDS,
// and the products of block p run while they arrive.
template <bool A_KC, bool B_KC, int KBT>
__global__ __launch_bounds__(512) void sdd_f32_tiled_kernel(
    const float *__restrict__ a, const float *__restrict__ b, float *__restrict__ c,
    const BlockDesc *__restrict__ blocks, const SchedEntry *__restrict__ sched,
    int n_swg, int batches, int nnz, int M, int N, int K)
{
    extern __shared__ __align__(16) unsigned char lds_raw[];
    int batch, swg;
    if (!map_workgroup(n_swg, batches, batch, swg)) return;
    const int w = wave_id(), l = lane_id();
    const int W = (int)(blockDim.x >> 6);
    const SchedEntry e = sched[swg * W + w];
    if (e.group < 0 || e.begin >= e.end) return;
    float *tiles = reinterpret_cast<float *>(lds_raw + (size_t)w * KBT * F32_TILE_BYTES);
    const float *ab = a + (size_t)batch * M * K;
    const float *bb = b + (size_t)batch * N * K;
    float *cb = c + (size_t)batch * nnz * BS2;
    const int r = e.group;

    uint4 raw[KBT][4];
    float aop[KBT][16];
    DescWindow win;
    const int first_end = e.begin + WAVE < e.end ? e.begin + WAVE : e.end;
    win.fetch(blocks, e.begin, first_end);
#pragma unroll
    for (int kb = 0; kb < KBT; ++kb) {
        if (A_KC) ldg_tile32_f32<false>(ab + (size_t)(BS * r) * K + BS * kb, K, raw[kb]);
        else ldg_tile32_f32<false>(ab + (size_t)(BS * kb) * M + BS * r, M, raw[kb]);
    }
    auto request = [&](int p) {
        const int cblk = win.get(p).col();
#pragma unroll
        for (int kb = 0; kb < KBT; ++kb) {
            if (B_KC) ldg_tile32_f32<false>(bb + (size_t)(BS * cblk) * K + BS * kb, K, raw[kb]);
            else ldg_tile32_f32<false>(bb + (size_t)(BS * kb) * N + BS * cblk, N, raw[kb]);
        }
    };
    auto park = [&]() {
        wave_lds_fence();
#pragma unroll
        for (int kb = 0; kb < KBT; ++kb) lds_put_f32(tiles + kb * (F32_TILE_BYTES / 4), raw[kb]);
        wave_lds_fence();
    };
    auto multiply = [&](int p) {
        f16v acc = {0};
#pragma unroll
        for (int kb = 0; kb < KBT; ++kb) {
            float bop[16];
            lds_get_f32<B_KC, true>(tiles + kb * (F32_TILE_BYTES / 4), bop);
#pragma unroll
            for (int t = 0; t < 16; ++t) acc = mfma_f32(bop[t], aop[kb][t], acc);
        }
        // a lane holds 16 consecutive columns of one row; the block leaves through LDS as four whole
        // kilobytes (64-byte pieces at 128-byte stride straight from the registers write at a third of the rate)
        wave_lds_fence();
#pragma unroll
        for (int q = 0; q < 4; ++q)
            *reinterpret_cast<float4 *>(tiles + get_f32_kc_addr(false, l, q) / 4) =
                make_float4(acc[4 * q], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]);
        wave_lds_fence();
        float *dst = cb + (size_t)win.get(p).idx * BS2;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            stg16_stream(dst + 4 * (l + 64 * j),
                         *reinterpret_cast<const uint4 *>(tiles + put_f32_addr(l, j) / 4));
    };
    park();
#pragma unroll
    for (int kb = 0; kb < KBT; ++kb) lds_get_f32<A_KC, false>(tiles + kb * (F32_TILE_BYTES / 4), aop[kb]);
    for (int seg = e.begin; seg < e.end; seg += WAVE) {
        const int seg_end = seg + WAVE < e.end ? seg + WAVE : e.end;
        if (seg != e.begin) win.fetch(blocks, seg, seg_end);
        request(seg);
        for (int p = seg; p + 1 < seg_end; ++p) {
            park();
            request(p + 1);
            multiply(p);
        }
        park();
        multiply(seg_end - 1);
    }
}

// ---------------------------------------------------------------------------
// Group walk (DSD and DDS).
//
//   out(x, y) = sum over the pairs of group g, sum over k of
//               Sblk(x, k) * Dn(32 * kblk + k, y)
//
// x = 0..31 runs inside the group's block row/column of the sparse matrix,
// y runs along the free dense dimension DN (a wave owns a strip of 64).
//   S_KC  the stored block is [x][k] (row groups, kblk = pair column);
//         otherwise [k][x] (column groups, kblk = pair row)
//   D_KC  the dense operand is stored [DN][KT]; otherwise [KT][DN]
//   DSD   output is [XT][DN] (y contiguous); otherwise (DDS) [DN][XT]
// ---------------------------------------------------------------------------
// Team reduction through LDS + the leader's check.  Returns true for the wave
// that has to store.  Every wave of the workgroup must call this once.  The
// accumulators are NT vectors of EV floats per lane (2 x 16 for the 32x32x16
// products, 8 x 4 for the 16x16x32 ones): 32 floats either way.
template <class V, int NT, int EV>
__device__ __forceinline__ bool team_reduce(V (&acc)[NT], const SchedEntry &e, int w, unsigned char *lds_raw)
{
    static_assert(NT * EV == 32, "a wave owns a 32 x 64 fp32 tile");
    const int l = lane_id();
    const int slot0 = e.first_wave(), nw = e.team_waves();
    const bool active = e.group >= 0;
    const bool leader = active && w == slot0;
    float *mine = reinterpret_cast<float *>(lds_raw + (size_t)w * GW_LDS_PER_WAVE);
    if (active && !leader) {
        wave_lds_fence();
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int v = 0; v < EV; ++v) mine[(t * EV + v) * WAVE + l] = acc[t][v];
    }
    __syncthreads();
    if (leader) {
        for (int o = 1; o < nw; ++o) {
            const float *other = reinterpret_cast<const float *>(lds_raw + (size_t)(w + o) * GW_LDS_PER_WAVE);
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int v = 0; v < EV; ++v) acc[t][v] += other[(t * EV + v) * WAVE + l];
        }
    }
    return leader;
}

// FULL: the dense dimension is a multiple of 64, every strip has both 32-wide halves: no per-lane
// condition on a load and no branch around a product, so the compiler can count the loads in flight
// (a load under a condition makes it wait for ALL of them before the first use) and can read all six
// operands of a block from LDS before the first of the four MFMAs instead of exposing the LDS latency
// four times.
template <bool S_KC, bool D_KC, bool DSD, int DEPTH, bool BF, bool FULL>
__global__ __launch_bounds__(512) void gw_f16_kernel(
    const half_t *__restrict__ sp, const half_t *__restrict__ dn, half_t *__restrict__ out,
    const BlockDesc *__restrict__ blocks, const SchedGroup *__restrict__ sched_groups,
    const SchedEntry *__restrict__ sched, SplitWorkspace ws,
    int n_swg, int batches, int nnz, int DN, int KT, int XT, int sp_shared, int idx_is_pos)
{
    extern __shared__ __align__(16) unsigned char lds_raw[];
    int batch, swg;
    if (!map_workgroup(n_swg, batches, batch, swg)) return;   // whole workgroup leaves together
    const int w = wave_id(), l = lane_id();
    const int W = (int)(blockDim.x >> 6);
    const SchedEntry e = sched[swg * W + w];
    const int y0 = 64 * (int)blockIdx.y;
    const int ytiles = FULL ? 2 : ((DN - y0) >= 64 ? 2 : 1);

    half_t *tile_s = reinterpret_cast<half_t *>(lds_raw + (size_t)w * GW_LDS_PER_WAVE);
    half_t *tile_d = tile_s + BS2;
    const half_t *spb = sp + (sp_shared ? 0 : (size_t)batch * nnz * BS2);   // one sparse operand for the whole batch?
    const half_t *dnb = dn + (size_t)batch * DN * KT;

    // one pair's operands: 2 KB of the sparse block + up to 4 KB of the dense strip,
    // every request fully coalesced
    struct Frag { uint4 s[2]; uint4 d0[2]; uint4 d1[2]; };

    DescWindow win;
    auto load_dense = [&](int p, Frag &f) {
        const BlockDesc d = win.get(p);
        const int kblk = S_KC ? d.col() : d.row();
        if (D_KC) {          // stored [DN][KT]: two 32 x 32 tiles, rows KT apart
            const half_t *src = dnb + (size_t)y0 * KT + BS * kblk;
            ldg_tile32(src, KT, f.d0);
            if (ytiles == 2) ldg_tile32(src + (size_t)32 * KT, KT, f.d1);
        } else {             // stored [KT][DN]: 32 rows of 64 (or 32) halves
            const half_t *src = dnb + (size_t)(BS * kblk) * DN + y0;
            const int pieces = 4 * ytiles;   // 16-byte pieces per k row
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                int cidx = l + 64 * q;
                int row = cidx >> 3, ch = cidx & 7;
                uint4 v = make_uint4(0, 0, 0, 0);
                if (FULL || ch < pieces) v = ldg16(src + (size_t)row * DN + 8 * ch);
                (q < 2 ? f.d0[q & 1] : f.d1[q & 1]) = v;
            }
        }
    };
    auto load = [&](int p, Frag &f) {
        ldg_block32_stream(spb + (size_t)win.get(p).idx * BS2, f.s);
        load_dense(p, f);
    };

    f16v acc[2] = {{0}, {0}};

    // DSD: the dense strip feeds the accumulator-register index (perm16), the block the lane index;
    // DDS: the other way round.
    auto compute = [&](const Frag &f) {
        wave_lds_fence();
        if (S_KC) lds_put_kc<!DSD>(tile_s, f.s);
        else lds_put_ks(tile_s, f.s);
        if (D_KC) {
            lds_put_kc<DSD>(tile_d, f.d0);
            if (ytiles == 2) lds_put_kc<DSD>(tile_d + BS2, f.d1);
        } else {
            lds_put_strip(tile_d, f.d0, f.d1);
        }
        wave_lds_fence();
        h8 sop[2], dop[2][2];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            sop[s] = S_KC ? lds_get_kc(tile_s, s) : lds_get_ks<!DSD>(tile_s, s);
#pragma unroll
            for (int t = 0; t < 2; ++t)
                if (t < ytiles)
                    dop[s][t] = D_KC ? lds_get_kc(tile_d + t * BS2, s) : lds_get_strip<DSD>(tile_d, 32 * t, s);
        }
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int t = 0; t < 2; ++t)
                if (t < ytiles) acc[t] = DSD ? mfma_16<BF>(dop[s][t], sop[s], acc[t]) : mfma_16<BF>(sop[s], dop[s][t], acc[t]);
    };

    if (e.group >= 0) {
        Frag fr[DEPTH];
        for (int seg = e.begin; seg < e.end; seg += WAVE) {
            const int seg_end = seg + WAVE < e.end ? seg + WAVE : e.end;
            win.fetch(blocks, seg, seg_end);
            int p = seg;
            if (seg_end - seg >= 2 * DEPTH) {
                // long enough for a steady state in which every load is unconditional.
                // In a row-major table pair p names block p, so the first block (from HBM, the longest
                // wait of the wave) is requested without waiting for the descriptors just asked for.
                if (idx_is_pos) {
                    ldg_block32_stream(spb + (size_t)seg * BS2, fr[0].s);
                    load_dense(seg, fr[0]);
                } else {
                    load(seg, fr[0]);
                }
#pragma unroll
                for (int d = 1; d < DEPTH; ++d) load(seg + d, fr[d]);
                for (; p + 2 * DEPTH <= seg_end; p += DEPTH) {
#pragma unroll
                    for (int d = 0; d < DEPTH; ++d) {
                        compute(fr[d]);
                        load(p + d + DEPTH, fr[d]);
                    }
                }
            } else {
#pragma unroll
                for (int d = 0; d < DEPTH; ++d)
                    if (seg + d < seg_end) load(seg + d, fr[d]);
            }
            for (; p < seg_end; p += DEPTH) {                // the last pairs: loads only while pairs are left
#pragma unroll
                for (int d = 0; d < DEPTH; ++d) {
                    if (p + d < seg_end) {
                        compute(fr[d]);
                        if (p + d + DEPTH < seg_end) load(p + d + DEPTH, fr[d]);
                    }
                }
            }
        }
    }

    const bool store_it = team_reduce<f16v, 2, 16>(acc, e, w, lds_raw) &&
                          (e.parts() <= 1 || split_combine<f16v, 2, 16>(acc, e, sched_groups[e.group], ws, batch));
    if (store_it) {
        half_t *ob = out + (size_t)batch * XT * DN;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            if (t < ytiles) {
                uint4 lo, hi;
                pack16<BF>(acc[t], lo, hi);
                half_t *o = ob + gw_out_offset<DSD>(e.group, y0, t, l, DN, XT);
                stg16(o, lo);
                stg16(o + 8, hi);
            }
        }
    }
}

// ---------------------------------------------------------------------------
// DSD over a ROW table with the dense operand stored [KT][DN] (the P V product of attention).
// The stored block is [x][k]: a lane's 8 halves of a 16 x 16 x 32 product (row x = lane % 16,
// k = 8 (lane / 16) ..) are 16 contiguous bytes of it, and the 64 lanes of one request cover 16
// whole rows = 1 KB of whole 128-byte lines.  The block therefore goes from global memory straight
// into operand registers (no LDS write, no LDS read); only the dense strip passes through LDS
// (put_strip16_addr / get_strip16_addr).  Accumulators: acc[4 xh + t] = rows 16 xh + lane % 16 of
// the block row, columns col16(t, 4 g + v).
// Pipeline: blocks come from HBM and are requested two steps ahead (two register sets of 8), strips
// come out of L2 and are requested one step ahead, right after the previous one has been copied to
// LDS (one register set of 16).  A wave's loads return in order, so strip p + 1 is requested BEFORE
// block p + 2.  104 registers less 16 against two full sets: the kernel fits four waves per SIMD,
// and a launch of about 3300 waves (seq 4096, 16 heads) is resident as a whole.
// ---------------------------------------------------------------------------
template <bool BF>
__global__ __launch_bounds__(512) void dsd_rows_f16_kernel(
    const half_t *__restrict__ sp, const half_t *__restrict__ dn, half_t *__restrict__ out,
    const BlockDesc *__restrict__ blocks, const SchedGroup *__restrict__ sched_groups,
    const SchedEntry *__restrict__ sched, SplitWorkspace ws,
    int n_swg, int batches, int nnz, int DN, int KT, int XT, int sp_shared)
{
    extern __shared__ __align__(16) unsigned char lds_raw[];
    int batch, swg;
    if (!map_workgroup(n_swg, batches, batch, swg)) return;   // whole workgroup leaves together
    const int w = wave_id(), l = lane_id();
    const int W = (int)(blockDim.x >> 6);
    const SchedEntry e = sched[swg * W + w];
    const int y0 = 64 * (int)blockIdx.y;
    const int g = l >> 4, i = l & 15;

    half_t *tile_d = reinterpret_cast<half_t *>(lds_raw + (size_t)w * GW_LDS_PER_WAVE);
    const half_t *spb = sp + (sp_shared ? 0 : (size_t)batch * nnz * BS2) + i * BS + 8 * g;
    const half_t *dnb = dn + (size_t)batch * DN * KT + y0;

    DescWindow win;
    uint4 blk[2][2], strip[4];
    auto issue_block = [&](int p, uint4 (&b)[2]) {             // pair p of a row table names block p
        const half_t *src = spb + (size_t)p * BS2;
        b[0] = ldg16_stream(src);
        b[1] = ldg16_stream(src + 16 * BS);
    };
    auto issue_strip = [&](int p) {
        const half_t *src = dnb + (size_t)(BS * win.get(p).col()) * DN;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int c = l + 64 * q;
            strip[q] = ldg16(src + (size_t)(c >> 3) * DN + 8 * (c & 7));
        }
    };

    f4v acc[8] = {{0}, {0}, {0}, {0}, {0}, {0}, {0}, {0}};
    half_t *ob = out + (size_t)batch * XT * DN + y0 + 8 * g;
    auto store_group = [&](int group) {
#pragma unroll
        for (int xh = 0; xh < 2; ++xh) {
            half_t *orow = ob + (size_t)(BS * group + 16 * xh + i) * DN;
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                h8 o;
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    o[v] = narrow_16<BF>(acc[4 * xh + 2 * u][v]);
                    o[4 + v] = narrow_16<BF>(acc[4 * xh + 2 * u + 1][v]);
                }
                stg16(orow + 32 * u, __builtin_bit_cast(uint4, o));
            }
        }
    };

    auto stage = [&]() {                      // the strip in flight -> LDS
        wave_lds_fence();
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            // rows 8-15 and 24-31 (q odd) are stored with the halves of every piece exchanged
            const uint4 v = (q & 1) ? make_uint4(strip[q].z, strip[q].w, strip[q].x, strip[q].y) : strip[q];
            *reinterpret_cast<uint4 *>(lds_bytes(tile_d) + put_strip16_addr(l, q)) = v;
        }
        wave_lds_fence();
    };
    auto multiply = [&](const uint4 (&b)[2]) {
        h8 dop[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            h4 lo = lds_read_tr16(reinterpret_cast<const half_t *>(lds_bytes(tile_d) + get_strip16_addr(l, t, 0)));
            h4 hi = lds_read_tr16(reinterpret_cast<const half_t *>(lds_bytes(tile_d) + get_strip16_addr(l, t, 1)));
            dop[t] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
#pragma unroll
        for (int xh = 0; xh < 2; ++xh)
#pragma unroll
            for (int t = 0; t < 4; ++t) acc[4 * xh + t] = mfma_16x16<BF>(dop[t], as_h8(b[xh]), acc[4 * xh + t]);
    };

    if (e.group >= 0) {
        for (int seg = e.begin; seg < e.end; seg += WAVE) {
            const int seg_end = seg + WAVE < e.end ? seg + WAVE : e.end;
            win.fetch(blocks, seg, seg_end);
            issue_block(seg, blk[0]);                 // from HBM, the longest wait: does not wait for the descriptors
            issue_strip(seg);
            int p = seg;
            if (seg + 3 < seg_end) {
                // steady state, two steps per round.  No load under a condition here nor on the way in: the
                // compiler's wait counts are only exact when every path into the loop has issued the same loads.
                issue_block(seg + 1, blk[1]);
                for (; p + 3 < seg_end; p += 2) {
                    stage();
                    issue_strip(p + 1);
                    multiply(blk[0]);
                    issue_block(p + 2, blk[0]);
                    stage();
                    issue_strip(p + 2);
                    multiply(blk[1]);
                    issue_block(p + 3, blk[1]);
                }
            } else if (seg + 1 < seg_end) {
                issue_block(seg + 1, blk[1]);
            }
            const int left = seg_end - p;             // 1, 2 or 3 pairs: blocks p and p + 1 and strip p are in flight
            stage();
            if (left >= 2) issue_strip(p + 1);
            multiply(blk[0]);
            if (left >= 3) issue_block(p + 2, blk[0]);
            if (left >= 2) {
                stage();
                if (left >= 3) issue_strip(p + 2);
                multiply(blk[1]);
            }
            if (left >= 3) {
                stage();
                multiply(blk[0]);
            }
        }
    }

    const bool store_it = team_reduce<f4v, 8, 4>(acc, e, w, lds_raw) &&
                          (e.parts() <= 1 || split_combine<f4v, 8, 4>(acc, e, sched_groups[e.group], ws, batch));
    if (store_it) store_group(e.group);
}

// ---------------------------------------------------------------------------
// DSD on a mask of 64 x 64 blocks, the block as the unit of work.  The operand is stored as the 2 x 2
// tiles of 32 x 32 of every block, in the row-major order of the mask with every cell repeated twice
// along both axes: block j of a coarse row r with n blocks, whose tiles start at base = 4 offsets[r],
// has its upper tiles at base + 2 j, + 1 and its lower ones 2 n further on.  A wave walks coarse pairs
// and takes, per 32 columns of the block, the upper and the lower tile (straight into operand registers,
// as in dsd_rows_f16_kernel) and ONE dense strip, staged once and multiplied into both: 8 KB of strips
// per 8 KB of block instead of 16 KB when the four tiles are walked as blocks of their own.
// Accumulators: 64 x 64 fp32 per wave.  Groups are never split across workgroups (the schedule must be
// built without BSA_SCHED_SPLIT); the waves of a team reduce through LDS.
// ---------------------------------------------------------------------------
constexpr int GW64_LDS_PER_WAVE = 16384;    // the strip (4 KB) while walking, the 64 x 64 fp32 partial tile afterwards

template <bool BF>
__global__ __launch_bounds__(256) void dsd_rows64_f16_kernel(
    const half_t *__restrict__ sp, const half_t *__restrict__ dn, half_t *__restrict__ out,
    const BlockDesc *__restrict__ blocks, const int *__restrict__ offsets, const SchedEntry *__restrict__ sched,
    int n_swg, int batches, int tiles, int DN, int KT, int XT, int sp_shared)
{
    extern __shared__ __align__(16) unsigned char lds_raw[];
    int batch, swg;
    if (!map_workgroup(n_swg, batches, batch, swg)) return;   // whole workgroup leaves together
    const int w = wave_id(), l = lane_id();
    const int W = (int)(blockDim.x >> 6);
    const SchedEntry e = sched[swg * W + w];
    const int y0 = 64 * (int)blockIdx.y;
    const int g = l >> 4, i = l & 15;

    half_t *tile_d = reinterpret_cast<half_t *>(lds_raw + (size_t)w * GW64_LDS_PER_WAVE);
    const half_t *spb = sp + (sp_shared ? 0 : (size_t)batch * tiles * BS2) + i * BS + 8 * g;
    const half_t *dnb = dn + (size_t)batch * DN * KT + y0;

    f4v acc[16];                       // acc[8 r + 4 xh + t]: tile row r (upper, lower), 16 block rows xh, columns col16(t, .)
#pragma unroll
    for (int t = 0; t < 16; ++t) acc[t] = f4v{0};

    if (e.group >= 0 && e.begin < e.end) {
        const int first = offsets[e.group], n = offsets[e.group + 1] - first;
        const size_t upper = (size_t)4 * first, lower = upper + (size_t)2 * n;      // tile index of column step 0
        DescWindow win;
        uint4 blk[2][4], strip[4];
        // column step s = 2 (pair - first) + half: the 32 columns `half` of the pair's block
        auto issue_block = [&](int s, uint4 (&b)[4]) {
            const half_t *up = spb + (upper + s) * BS2, *lo = spb + (lower + s) * BS2;
            b[0] = ldg16_stream(up);
            b[1] = ldg16_stream(up + 16 * BS);
            b[2] = ldg16_stream(lo);
            b[3] = ldg16_stream(lo + 16 * BS);
        };
        auto issue_strip = [&](int s) {
            const int col32 = 2 * win.get(first + (s >> 1)).col() + (s & 1);
            const half_t *src = dnb + (size_t)(BS * col32) * DN;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int c = l + 64 * q;
                strip[q] = ldg16(src + (size_t)(c >> 3) * DN + 8 * (c & 7));
            }
        };
        auto stage = [&]() {
            wave_lds_fence();
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint4 v = (q & 1) ? make_uint4(strip[q].z, strip[q].w, strip[q].x, strip[q].y) : strip[q];
                *reinterpret_cast<uint4 *>(lds_bytes(tile_d) + put_strip16_addr(l, q)) = v;
            }
            wave_lds_fence();
        };
        auto multiply = [&](const uint4 (&b)[4]) {
            h8 dop[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                h4 lo = lds_read_tr16(reinterpret_cast<const half_t *>(lds_bytes(tile_d) + get_strip16_addr(l, t, 0)));
                h4 hi = lds_read_tr16(reinterpret_cast<const half_t *>(lds_bytes(tile_d) + get_strip16_addr(l, t, 1)));
                dop[t] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
#pragma unroll
            for (int r = 0; r < 2; ++r)
#pragma unroll
                for (int xh = 0; xh < 2; ++xh)
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        acc[8 * r + 4 * xh + t] = mfma_16x16<BF>(dop[t], as_h8(b[2 * r + xh]), acc[8 * r + 4 * xh + t]);
        };
        for (int seg = e.begin; seg < e.end; seg += WAVE) {
            const int seg_end = seg + WAVE < e.end ? seg + WAVE : e.end;
            win.fetch(blocks, seg, seg_end);
            int s = 2 * (seg - first);
            const int s_end = 2 * (seg_end - first), last = s_end - 1;     // an even number of column steps
            issue_block(s, blk[0]);
            issue_strip(s);
            issue_block(s + 1, blk[1]);
            // Two steps per round and no load under a condition: behind the last step the requests repeat it
            // (served by the caches, never used), which keeps ONE copy of the loop body and exact wait counts.
            for (; s < s_end; s += 2) {
                stage();
                issue_strip(s + 1);
                multiply(blk[0]);
                issue_block(s + 2 < last ? s + 2 : last, blk[0]);
                stage();
                issue_strip(s + 2 < last ? s + 2 : last);
                multiply(blk[1]);
                issue_block(s + 3 < last ? s + 3 : last, blk[1]);
            }
        }
    }

    // team reduction through LDS: every wave of the workgroup arrives here once
    const int slot0 = e.first_wave(), nw = e.team_waves();
    const bool active = e.group >= 0;
    const bool leader = active && w == slot0;
    float *mine = reinterpret_cast<float *>(lds_raw + (size_t)w * GW64_LDS_PER_WAVE);
    if (active && !leader) {
        wave_lds_fence();
#pragma unroll
        for (int t = 0; t < 16; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) mine[(t * 4 + v) * WAVE + l] = acc[t][v];
    }
    __syncthreads();
    if (!leader) return;
    for (int o = 1; o < nw; ++o) {
        const float *other = reinterpret_cast<const float *>(lds_raw + (size_t)(w + o) * GW64_LDS_PER_WAVE);
#pragma unroll
        for (int t = 0; t < 16; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[t][v] += other[(t * 4 + v) * WAVE + l];
    }
    half_t *ob = out + (size_t)batch * XT * DN + y0 + 8 * g;
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int xh = 0; xh < 2; ++xh) {
            half_t *orow = ob + (size_t)(64 * e.group + 32 * r + 16 * xh + i) * DN;
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                h8 o;
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    o[v] = narrow_16<BF>(acc[8 * r + 4 * xh + 2 * u][v]);
                    o[4 + v] = narrow_16<BF>(acc[8 * r + 4 * xh + 2 * u + 1][v]);
                }
                stg16(orow + 32 * u, __builtin_bit_cast(uint4, o));
            }
        }
}

template <bool S_KC, bool D_KC, bool DSD>
__global__ __launch_bounds__(512) void gw_f32_kernel(
    const float *__restrict__ sp, const float *__restrict__ dn, float *__restrict__ out,
    const BlockDesc *__restrict__ blocks, const SchedGroup *__restrict__ sched_groups,
    const SchedEntry *__restrict__ sched, SplitWorkspace ws,
    int n_swg, int batches, int nnz, int DN, int KT, int XT, int sp_shared)
{
    extern __shared__ __align__(16) unsigned char lds_raw[];
    int batch, swg;
    if (!map_workgroup(n_swg, batches, batch, swg)) return;
    const int w = wave_id(), l = lane_id();
    const int W = (int)(blockDim.x >> 6);
    const SchedEntry e = sched[swg * W + w];
    const int y0 = 64 * (int)blockIdx.y;
    const int ytiles = (DN - y0) >= 64 ? 2 : 1;
    const float *spb = sp + (sp_shared ? 0 : (size_t)batch * nnz * BS2);
    const float *dnb = dn + (size_t)batch * DN * KT;

    f16v acc[2] = {{0}, {0}};
    if (e.group >= 0) {
        DescWindow win;
        for (int p = e.begin; p < e.end; ++p) {
            if (((p - e.begin) & (WAVE - 1)) == 0) win.fetch(blocks, p, e.end);
            const BlockDesc d = win.get(p);
            const int kblk = S_KC ? d.col() : d.row();
            float sv[16], dv[2][16];
            ldg_tile_f32<S_KC, !DSD>(spb + (size_t)d.idx * BS2, BS, sv);
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                if (t < ytiles) {
                    if (D_KC) ldg_tile_f32<true, DSD>(dnb + (size_t)(y0 + 32 * t) * KT + BS * kblk, KT, dv[t]);
                    else ldg_tile_f32<false, DSD>(dnb + (size_t)(BS * kblk) * DN + y0 + 32 * t, DN, dv[t]);
                }
            }
#pragma unroll
            for (int k = 0; k < 16; ++k) {
                if (DSD) {
                    acc[0] = mfma_f32(dv[0][k], sv[k], acc[0]);
                    if (ytiles == 2) acc[1] = mfma_f32(dv[1][k], sv[k], acc[1]);
                } else {
                    acc[0] = mfma_f32(sv[k], dv[0][k], acc[0]);
                    if (ytiles == 2) acc[1] = mfma_f32(sv[k], dv[1][k], acc[1]);
                }
            }
        }
    }
    if (team_reduce<f16v, 2, 16>(acc, e, w, lds_raw) &&
        (e.parts() <= 1 || split_combine<f16v, 2, 16>(acc, e, sched_groups[e.group], ws, batch))) {
        float *ob = out + (size_t)batch * XT * DN;
#pragma unroll
        for (int t = 0; t < 2; ++t)
            if (t < ytiles) store16_f32(ob + gw_out_offset<DSD>(e.group, y0, t, l, DN, XT), acc[t]);
    }
}

// The same walk for a dense dimension that is a multiple of 64, with every operand tile fetched by coalesced
// requests and turned into MFMA operands through the wave's LDS tile (one tile at a time: the partial-tile
// area of the team reduce is enough), and with the three tiles of pair p + 1 requested before the 32 products
// of pair p are issued.
template <bool S_KC, bool D_KC, bool DSD>
__global__ __launch_bounds__(512) void gw_f32_tiled_kernel(
    const float *__restrict__ sp, const float *__restrict__ dn, float *__restrict__ out,
    const BlockDesc *__restrict__ blocks, const SchedGroup *__restrict__ sched_groups,
    const SchedEntry *__restrict__ sched, SplitWorkspace ws,
    int n_swg, int batches, int nnz, int DN, int KT, int XT, int sp_shared)
{
    extern __shared__ __align__(16) unsigned char lds_raw[];
    static_assert(F32_TILE_BYTES <= GW_LDS_PER_WAVE, "the operand tile shares the wave's reduce area");
    int batch, swg;
    if (!map_workgroup(n_swg, batches, batch, swg)) return;
    const int w = wave_id(), l = lane_id();
    const int W = (int)(blockDim.x >> 6);
    const SchedEntry e = sched[swg * W + w];
    const int y0 = 64 * (int)blockIdx.y;
    const float *spb = sp + (sp_shared ? 0 : (size_t)batch * nnz * BS2);
    const float *dnb = dn + (size_t)batch * DN * KT;
    float *tile = reinterpret_cast<float *>(lds_raw + (size_t)w * GW_LDS_PER_WAVE);

    f16v acc[2] = {{0}, {0}};
    if (e.group >= 0) {
        DescWindow win;
        uint4 sraw[4], draw[2][4];
        auto request = [&](int p) {
            const BlockDesc d = win.get(p);
            const int kblk = S_KC ? d.col() : d.row();
            ldg_tile32_f32<true>(spb + (size_t)d.idx * BS2, BS, sraw);
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                if (D_KC) ldg_tile32_f32<false>(dnb + (size_t)(y0 + 32 * t) * KT + BS * kblk, KT, draw[t]);
                else ldg_tile32_f32<false>(dnb + (size_t)(BS * kblk) * DN + y0 + 32 * t, DN, draw[t]);
            }
        };
        auto operands = [&](float (&sv)[16], float (&dv)[2][16]) {
            wave_lds_fence();
            lds_put_f32(tile, sraw);
            wave_lds_fence();
            lds_get_f32<S_KC, !DSD>(tile, sv);
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                wave_lds_fence();
                lds_put_f32(tile, draw[t]);
                wave_lds_fence();
                lds_get_f32<D_KC, DSD>(tile, dv[t]);
            }
        };
        auto multiply = [&](const float (&sv)[16], const float (&dv)[2][16]) {
#pragma unroll
            for (int k = 0; k < 16; ++k) {
                if (DSD) {
                    acc[0] = mfma_f32(dv[0][k], sv[k], acc[0]);
                    acc[1] = mfma_f32(dv[1][k], sv[k], acc[1]);
                } else {
                    acc[0] = mfma_f32(sv[k], dv[0][k], acc[0]);
                    acc[1] = mfma_f32(sv[k], dv[1][k], acc[1]);
                }
            }
        };
        for (int seg = e.begin; seg < e.end; seg += WAVE) {
            const int seg_end = seg + WAVE < e.end ? seg + WAVE : e.end;
            win.fetch(blocks, seg, seg_end);
            request(seg);
            float sv[16], dv[2][16];
            for (int p = seg; p + 1 < seg_end; ++p) {
                operands(sv, dv);
                request(p + 1);
                multiply(sv, dv);
            }
            operands(sv, dv);
            multiply(sv, dv);
        }
        wave_lds_fence();    // the tile area becomes the wave's partial tile below
    }
    if (team_reduce<f16v, 2, 16>(acc, e, w, lds_raw) &&
        (e.parts() <= 1 || split_combine<f16v, 2, 16>(acc, e, sched_groups[e.group], ws, batch))) {
        float *ob = out + (size_t)batch * XT * DN;
#pragma unroll
        for (int t = 0; t < 2; ++t) store16_f32(ob + gw_out_offset<DSD>(e.group, y0, t, l, DN, XT), acc[t]);
    }
}

// ---------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------
static inline unsigned grid_x(int n_swg, int batches) { return 8u * (unsigned)n_swg * (unsigned)((batches + 7) / 8); }
static inline const SchedGroup *sched_groups(const MatmulArgs &p) { return (const SchedGroup *)p.sched; }
static inline const SchedEntry *sched_slots(const MatmulArgs &p) { return (const SchedEntry *)p.sched + p.groups; }

template <bool A_KC, bool B_KC, bool BF>
static hipError_t launch_sdd_f16(const MatmulArgs &p, hipStream_t st)
{
    dim3 grid(grid_x(p.sched_wgs, p.batches)), block(64 * p.sched_waves);
    size_t lds = (size_t)p.sched_waves * SDD_LDS_PER_WAVE;
#define BSA_SDD_ARGS (const half_t *)p.a, (const half_t *)p.b, (half_t *)p.c, (const BlockDesc *)p.blocks, \
                     sched_slots(p), p.sched_wgs, p.batches, p.nnz, p.M, p.N, p.K
    switch (p.K / BS) {
        case 1: sdd_f16_kernel<A_KC, B_KC, 1, BF><<<grid, block, lds, st>>>(BSA_SDD_ARGS); break;
        case 2: sdd_f16_kernel<A_KC, B_KC, 2, BF><<<grid, block, lds, st>>>(BSA_SDD_ARGS); break;
        case 3: sdd_f16_kernel<A_KC, B_KC, 3, BF><<<grid, block, lds, st>>>(BSA_SDD_ARGS); break;
        case 4: sdd_f16_kernel<A_KC, B_KC, 4, BF><<<grid, block, lds, st>>>(BSA_SDD_ARGS); break;
        default: sdd_f16_kernel<A_KC, B_KC, 0, BF><<<grid, block, lds, st>>>(BSA_SDD_ARGS); break;
    }
#undef BSA_SDD_ARGS
    return hipGetLastError();
}

template <bool A_KC, bool B_KC>
static hipError_t launch_sdd_f32(const MatmulArgs &p, hipStream_t st)
{
    dim3 grid(grid_x(p.sched_wgs, p.batches)), block(64 * p.sched_waves);
#define BSA_SDD_ARGS (const float *)p.a, (const float *)p.b, (float *)p.c, (const BlockDesc *)p.blocks, \
                     sched_slots(p), p.sched_wgs, p.batches, p.nnz, p.M, p.N, p.K
    const int kbs = p.K / BS;
    const size_t lds = (size_t)p.sched_waves * kbs * F32_TILE_BYTES;
    if (kbs <= 4 && lds <= 163840) {      // at most 8 waves x 4 tiles of 4864 bytes: a compute unit's 160 KB hold it
        auto launch = [&](auto kernel) {
            hipError_t err = hipSuccess;
            if (lds > 65536)
                err = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (err != hipSuccess) return err;
            kernel<<<grid, block, lds, st>>>(BSA_SDD_ARGS);
            return hipGetLastError();
        };
        switch (kbs) {
            case 1: return launch(sdd_f32_tiled_kernel<A_KC, B_KC, 1>);
            case 2: return launch(sdd_f32_tiled_kernel<A_KC, B_KC, 2>);
            case 3: return launch(sdd_f32_tiled_kernel<A_KC, B_KC, 3>);
            default: return launch(sdd_f32_tiled_kernel<A_KC, B_KC, 4>);
        }
    }
    sdd_f32_kernel<A_KC, B_KC><<<grid, block, 0, st>>>(BSA_SDD_ARGS);
#undef BSA_SDD_ARGS
    return hipGetLastError();
}

hipError_t launch_sdd(int dtype, const MatmulArgs &p, hipStream_t st)
{
    // op(a) is M x K: stored [M][K] (contraction contiguous) unless tr_a.
    // op(b) is K x N: stored [N][K] (contraction contiguous) only with tr_b.
    const bool a_kc = !p.tr_a, b_kc = p.tr_b;
    if (dtype == BSA_F16) {
        if (a_kc) return b_kc ? launch_sdd_f16<true, true, false>(p, st) : launch_sdd_f16<true, false, false>(p, st);
        return b_kc ? launch_sdd_f16<false, true, false>(p, st) : launch_sdd_f16<false, false, false>(p, st);
    }
    if (dtype == BSA_BF16) {
        if (a_kc) return b_kc ? launch_sdd_f16<true, true, true>(p, st) : launch_sdd_f16<true, false, true>(p, st);
        return b_kc ? launch_sdd_f16<false, true, true>(p, st) : launch_sdd_f16<false, false, true>(p, st);
    }
    if (a_kc) return b_kc ? launch_sdd_f32<true, true>(p, st) : launch_sdd_f32<true, false>(p, st);
    return b_kc ? launch_sdd_f32<false, true>(p, st) : launch_sdd_f32<false, false>(p, st);
}

template <bool S_KC, bool D_KC, bool DSD>
static hipError_t launch_gw_t(int dtype, const void *sp, const void *dn, const MatmulArgs &p,
                              int DN, int KT, int XT, hipStream_t st)
{
    dim3 grid(grid_x(p.sched_wgs, p.batches), (unsigned)((DN + 63) / 64)), block(64 * p.sched_waves);
    size_t lds = (size_t)p.sched_waves * GW_LDS_PER_WAVE;
    // workspace: counters of every (batch, strip, split group), then the partial tiles
    SplitWorkspace ws;
    ws.tile_slots = p.tile_slots;
    ws.split_groups = p.split_groups;
    ws.counters = (int *)p.workspace;
    ws.tiles = (float *)((char *)p.workspace + gw_counter_bytes(p.split_groups, p.batches, DN));
#define BSA_GW_ARGS (const half_t *)sp, (const half_t *)dn, (half_t *)p.c, (const BlockDesc *)p.blocks, \
                    sched_groups(p), sched_slots(p), ws, p.sched_wgs, p.batches, p.nnz, DN, KT, XT, p.sparse_shared ? 1 : 0, \
                    p.row_table ? 1 : 0
    const bool full = DN % 64 == 0;
    if (S_KC && !D_KC && DSD && full && p.row_table && dtype != BSA_F32) {
#define BSA_DR_ARGS (const half_t *)sp, (const half_t *)dn, (half_t *)p.c, (const BlockDesc *)p.blocks, \
                    sched_groups(p), sched_slots(p), ws, p.sched_wgs, p.batches, p.nnz, DN, KT, XT, p.sparse_shared ? 1 : 0
        if (dtype == BSA_F16) dsd_rows_f16_kernel<false><<<grid, block, lds, st>>>(BSA_DR_ARGS);
        else dsd_rows_f16_kernel<true><<<grid, block, lds, st>>>(BSA_DR_ARGS);
#undef BSA_DR_ARGS
        return hipGetLastError();
    }
    if (dtype == BSA_F16) {
        if (full) gw_f16_kernel<S_KC, D_KC, DSD, GW_PREFETCH_DEPTH, false, true><<<grid, block, lds, st>>>(BSA_GW_ARGS);
        else gw_f16_kernel<S_KC, D_KC, DSD, GW_PREFETCH_DEPTH, false, false><<<grid, block, lds, st>>>(BSA_GW_ARGS);
    } else if (dtype == BSA_BF16) {
        if (full) gw_f16_kernel<S_KC, D_KC, DSD, GW_PREFETCH_DEPTH, true, true><<<grid, block, lds, st>>>(BSA_GW_ARGS);
        else gw_f16_kernel<S_KC, D_KC, DSD, GW_PREFETCH_DEPTH, true, false><<<grid, block, lds, st>>>(BSA_GW_ARGS);
    } else
#undef BSA_GW_ARGS
    {
#define BSA_GW32_ARGS (const float *)sp, (const float *)dn, (float *)p.c, (const BlockDesc *)p.blocks, \
                      sched_groups(p), sched_slots(p), ws, p.sched_wgs, p.batches, p.nnz, DN, KT, XT, p.sparse_shared ? 1 : 0
        if (full) gw_f32_tiled_kernel<S_KC, D_KC, DSD><<<grid, block, lds, st>>>(BSA_GW32_ARGS);
        else gw_f32_kernel<S_KC, D_KC, DSD><<<grid, block, lds, st>>>(BSA_GW32_ARGS);
#undef BSA_GW32_ARGS
    }
    return hipGetLastError();
}

hipError_t launch_dsd_block64(int dtype, const Block64Args &p, hipStream_t st)
{
    dim3 grid(grid_x(p.sched_wgs, p.batches), (unsigned)(p.N / 64)), block(64 * p.sched_waves);
    const size_t lds = (size_t)p.sched_waves * GW64_LDS_PER_WAVE;
    const SchedEntry *slots = (const SchedEntry *)p.sched + p.coarse_rows;
    hipError_t err = hipSuccess;
    if (dtype == BSA_F16) {
        if (lds > 65536) err = hipFuncSetAttribute(reinterpret_cast<const void *>(dsd_rows64_f16_kernel<false>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (err != hipSuccess) return err;
        dsd_rows64_f16_kernel<false><<<grid, block, lds, st>>>(
            (const half_t *)p.a, (const half_t *)p.b, (half_t *)p.c, (const BlockDesc *)p.blocks, p.offsets, slots,
            p.sched_wgs, p.batches, 4 * p.coarse_nnz, p.N, 64 * p.coarse_cols, 64 * p.coarse_rows, p.sparse_shared ? 1 : 0);
    } else {
        if (lds > 65536) err = hipFuncSetAttribute(reinterpret_cast<const void *>(dsd_rows64_f16_kernel<true>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (err != hipSuccess) return err;
        dsd_rows64_f16_kernel<true><<<grid, block, lds, st>>>(
            (const half_t *)p.a, (const half_t *)p.b, (half_t *)p.c, (const BlockDesc *)p.blocks, p.offsets, slots,
            p.sched_wgs, p.batches, 4 * p.coarse_nnz, p.N, 64 * p.coarse_cols, 64 * p.coarse_rows, p.sparse_shared ? 1 : 0);
    }
    return hipGetLastError();
}

size_t gw_counter_bytes(int split_groups, int batches, int free_dim)
{
    size_t n = (size_t)split_groups * batches * ((free_dim + 63) / 64) * sizeof(int);
    return (n + 255) / 256 * 256;
}

size_t gw_workspace_bytes(int tile_slots, int split_groups, int batches, int free_dim)
{
    return gw_counter_bytes(split_groups, batches, free_dim) +
           (size_t)tile_slots * batches * ((free_dim + 63) / 64) * 2048 * sizeof(float);
}

// ---------------------------------------------------------------------------
// The group walk on the library's own scratch buffer, for callers that cannot allocate.
// `scratch` is device memory of this code object: every GPU the library runs on holds its own
// copy, at its own address, until the process ends.  In host code the NAME of the array is not a
// device address; the address is asked for once per device (hipGetSymbolAddress) and kept.
// ---------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[BSA_STATIC_SCRATCH_BYTES];

namespace {
constexpr int MAX_DEVICES = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[MAX_DEVICES] = {nullptr};

// The array of the device that holds `on_device` (the result of the call): each GPU has its own copy, and the
// caller's current device need not be the one its pointers live on.
hipError_t static_scratch(const void *on_device, void **ptr)
{
    hipPointerAttribute_t attr;
    hipError_t err = hipPointerGetAttributes(&attr, on_device);
    if (err != hipSuccess) return err;
    const int dev = attr.device;
    if (dev < 0 || dev >= MAX_DEVICES) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        int current = -1;
        err = hipGetDevice(&current);
        if (err != hipSuccess) return err;
        if (current != dev && (err = hipSetDevice(dev)) != hipSuccess) return err;
        void *p = nullptr;
        err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (current != dev) (void)hipSetDevice(current);
        if (err != hipSuccess) return err;
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return hipSuccess;
}
}  // namespace

__global__ void clear_ints_kernel(int *p, size_t n)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

hipError_t launch_group_walk_static_scratch(int dtype, bool dsd, const MatmulArgs &args, hipStream_t st)
{
    MatmulArgs p = args;
    p.workspace = nullptr;
    const int free_dim = dsd ? p.N : p.M;
    const size_t need = p.tile_slots > 0 ? gw_workspace_bytes(p.tile_slots, p.split_groups, p.batches, free_dim) : 0;
    if (need > (size_t)BSA_STATIC_SCRATCH_BYTES) return hipErrorOutOfMemory;   // the C ABI checks first and says why
    if (need > 0) {
        void *base = nullptr;
        hipError_t err = static_scratch(p.c, &base);
        if (err != hipSuccess) return err;
        // the counters must start at zero and the buffer keeps what the last call left (an earlier launch
        // may have failed midway); a kernel clears them, so that the call can sit in a captured graph
        const size_t ints = gw_counter_bytes(p.split_groups, p.batches, free_dim) / sizeof(int);
        clear_ints_kernel<<<(unsigned)((ints + 255) / 256), 256, 0, st>>>((int *)base, ints);
        err = hipGetLastError();
        if (err != hipSuccess) return err;
        p.workspace = base;
    }
    return launch_group_walk(dtype, dsd, p, st);
}

hipError_t launch_group_walk(int dtype, bool dsd, const MatmulArgs &p, hipStream_t st)
{
    if (dsd) {
        // sparse = a; row groups (stored block is [x][k]) unless tr_a.
        // dense = b, op(b) is K x N: stored [K][N] unless tr_b -> D_KC = tr_b.
        const bool s_kc = !p.tr_a, d_kc = p.tr_b;
        const int DN = p.N, KT = p.K, XT = p.M;
        if (s_kc) return d_kc ? launch_gw_t<true, true, true>(dtype, p.a, p.b, p, DN, KT, XT, st)
                              : launch_gw_t<true, false, true>(dtype, p.a, p.b, p, DN, KT, XT, st);
        return d_kc ? launch_gw_t<false, true, true>(dtype, p.a, p.b, p, DN, KT, XT, st)
                    : launch_gw_t<false, false, true>(dtype, p.a, p.b, p, DN, KT, XT, st);
    }
    // DDS: sparse = b; column groups (stored block is [k][x]) unless tr_b.
    // dense = a, op(a) is M x K: stored [M][K] unless tr_a -> D_KC = !tr_a.
    const bool s_kc = p.tr_b, d_kc = !p.tr_a;
    const int DN = p.M, KT = p.K, XT = p.N;
    if (s_kc) return d_kc ? launch_gw_t<true, true, false>(dtype, p.b, p.a, p, DN, KT, XT, st)
                          : launch_gw_t<true, false, false>(dtype, p.b, p.a, p, DN, KT, XT, st);
    return d_kc ? launch_gw_t<false, true, false>(dtype, p.b, p.a, p, DN, KT, XT, st)
                : launch_gw_t<false, false, false>(dtype, p.b, p.a, p, DN, KT, XT, st);
}


}  // namespace bsa
