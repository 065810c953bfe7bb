// Device-side builder of the block-index tables and of the wavefront schedule.
//
// Tables: the contract is the output of SparseLayout._create_layout
// (sparse/layout.py:14-38) for a 0/1 mask, both orientations.  One workgroup
// of 16 wavefronts scans the mask twice (row-major, then column-major) with
// wave ballots + popcounts; the row-major ordinal of every cell is parked in a
// workspace so the column pass can attach it to its pairs.
//
// Schedule: see bsa.h.  A serial first-fit pass over the groups (one lane)
// fixes each group's first slot and its partial-tile slots, then all lanes
// fill the wavefront slots.
#include "bsa_device.hpp"
#include "bsa_internal.hpp"
#include "../../include/bsa.h"

namespace bsa {

constexpr int LB_THREADS = 1024;
constexpr int LB_WAVES = LB_THREADS / WAVE;

// Exclusive position of this thread's flag among the flags of the workgroup,
// and the workgroup total.  `carry` is the running count of earlier tiles.
__device__ __forceinline__ int tile_scan(bool flag, int *wave_tot, int &total)
{
    unsigned long long bal = __ballot(flag);
    int lane = lane_id(), wave = (int)(threadIdx.x >> 6);
    int lane_prefix = __popcll(bal & ((1ull << lane) - 1ull));
    if (lane == 0) wave_tot[wave] = __popcll(bal);
    __syncthreads();
    int wave_prefix = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < LB_WAVES; ++w) {
        int t = wave_tot[w];
        wave_prefix += (w < wave) ? t : 0;
        tot += t;
    }
    __syncthreads();
    total = tot;
    return wave_prefix + lane_prefix;
}

__global__ __launch_bounds__(LB_THREADS) void layout_build_kernel(
    const uint8_t *__restrict__ mask, int R, int C,
    int2 *__restrict__ row_blocks, int *__restrict__ row_off,
    int2 *__restrict__ col_blocks, int *__restrict__ col_off,
    int *__restrict__ nnz_out, int *__restrict__ ordinal_of)
{
    __shared__ int wave_tot[LB_WAVES];
    const int n = R * C;
    const int tid = (int)threadIdx.x;

    // pass 1: row-major order -> row table, ordinals
    int carry = 0;
    for (int base = 0; base < n; base += LB_THREADS) {
        int t = base + tid;
        bool nz = t < n && mask[t] != 0;
        int total;
        int ord = carry + tile_scan(nz, wave_tot, total);
        if (t < n) {
            int r = t / C, c = t - r * C;
            ordinal_of[t] = ord;
            if (c == 0) row_off[r] = ord;
            if (nz) row_blocks[ord] = make_int2(ord, (int)(((unsigned)r << 16) + (unsigned)c));
        }
        carry += total;
    }
    if (tid == 0) {
        row_off[R] = carry;
        col_off[C] = carry;
        nnz_out[0] = carry;
    }
    __syncthreads();   // ordinal_of is re-read below by other lanes of this workgroup

    // pass 2: column-major order -> column table
    carry = 0;
    for (int base = 0; base < n; base += LB_THREADS) {
        int t = base + tid;
        int c = t / R, r = t - c * R;
        int cell = r * C + c;
        bool nz = t < n && mask[cell] != 0;
        int total;
        int pos = carry + tile_scan(nz, wave_tot, total);
        if (t < n) {
            if (r == 0) col_off[c] = pos;
            if (nz) col_blocks[pos] = make_int2(ordinal_of[cell], (int)(((unsigned)r << 16) + (unsigned)c));
        }
        carry += total;
    }
}

// ---- schedule -------------------------------------------------------------
// Buffer layout (int4 units): [0, groups) per-group meta, then the wavefront slots.
//   meta[g] = (first slot of part 0, first partial-tile slot or -1, ordinal among split groups or -1, parts)

struct GroupPlan {
    int parts;      // workgroup-sized pieces the group is cut into (or row slices, see below)
    int len;
    bool sliced;    // the whole group goes to `slices` waves, each taking 32 / slices of its element rows
};

__device__ __forceinline__ GroupPlan plan_group(int len, int cap, int waves, int allow_split, int slice_max, int slices)
{
    GroupPlan p;
    p.len = len;
    p.sliced = len <= slice_max;
    if (p.sliced) {
        p.parts = slices;
        return p;
    }
    const int span = cap * waves;                       // pairs one workgroup takes at the target chunk size
    int parts = allow_split ? (len + span - 1) / span : 1;
    parts = parts < 1 ? 1 : (parts > SCHED_MAX_PARTS ? SCHED_MAX_PARTS : parts);
    p.parts = parts;
    return p;
}

// pairs [lo, hi) of piece t out of n of a range of `len`
__device__ __forceinline__ int piece_lo(int len, int t, int n) { return (int)(((long long)len * t) / n); }

__device__ __forceinline__ int waves_of_part(int part_len, int cap, int waves)
{
    int nw = (part_len + cap - 1) / cap;
    nw = nw < 1 ? 1 : nw;
    return nw > waves ? waves : nw;
}

__global__ __launch_bounds__(LB_THREADS) void schedule_build_kernel(
    const int *__restrict__ offsets, int groups, int cap, int waves, int flags, int slice_max, int slices,
    int4 *__restrict__ sched, int slot_capacity, int *__restrict__ counts_out)
{
    const int allow_split = flags & BSA_SCHED_SPLIT;
    const bool longest_first = (flags & BSA_SCHED_LONGEST_FIRST) != 0;
    __shared__ int total_slots;
    const int tid = (int)threadIdx.x;
    int4 *meta = sched;
    int4 *slots = sched + groups;
    // Serial first-fit, one pass over the groups per class.  Row-sliced groups fill whole workgroups of
    // their own (their waves need no barrier).  Split groups come before the unsplit ones: their parts
    // meet in a workspace after the walk, and workgroups are dispatched in slot order, so starting them
    // first lets that exchange run while the rest of the launch is still multiplying.
    // Without BSA_SCHED_LONGEST_FIRST: sliced, split, unsplit, each in table order.  With it, long work
    // starts first: split groups, then the unsplit ones by their longest chunk (quarters of cap), then the
    // sliced ones (all shorter than any other group) by length (quarters of the longest of them).  A wave
    // walks its chunk serially and a launch of these kernels is only one or two rounds of waves, so a long
    // chunk that starts last (the late rows of a causal mask) runs on an almost empty machine.
    // A team (the waves of one part) never straddles a workgroup boundary.
    if (tid == 0) {
        int pos = 0, tile_slots = 0, split_groups = 0;
        constexpr int LEN_CLASSES = 4;     // by length: > 3/4, > 1/2, > 1/4 of the yardstick, rest
        constexpr int CLS_SLICED = 0, CLS_SPLIT = LEN_CLASSES, CLS_UNSPLIT = LEN_CLASSES + 1;
        int longest_sliced = 0;
        if (longest_first)
            for (int g = 0; g < groups; ++g) {
                const int len = offsets[g + 1] - offsets[g];
                if (len <= slice_max && len > longest_sliced) longest_sliced = len;
            }
        auto len_class = [](int len, int yard) {
            return 4 * len > 3 * yard ? 0 : (2 * len > yard ? 1 : (4 * len > yard ? 2 : 3));
        };
        const int n_pass = longest_first ? 1 + 2 * LEN_CLASSES : 3;
        for (int pass = 0; pass < n_pass; ++pass) {
            // class handled by this pass
            const int want = longest_first ? (pass <= LEN_CLASSES ? CLS_SPLIT + pass : pass - LEN_CLASSES - 1)
                                           : (pass == 0 ? CLS_SLICED : CLS_SPLIT + pass - 1);
            // the sliced region starts (and ends) on a workgroup boundary
            if (want == CLS_SLICED || (!longest_first && want == CLS_SPLIT)) pos = (pos + waves - 1) / waves * waves;
            for (int g = 0; g < groups; ++g) {
                const GroupPlan gp = plan_group(offsets[g + 1] - offsets[g], cap, waves, allow_split, slice_max, slices);
                int cls;
                if (gp.sliced) {
                    cls = CLS_SLICED + (longest_first ? len_class(gp.len, longest_sliced) : 0);
                } else if (gp.parts > 1) {
                    cls = CLS_SPLIT;
                } else {
                    cls = CLS_UNSPLIT;
                    if (longest_first) {
                        const int nw = waves_of_part(gp.len, cap, waves);
                        cls += len_class((gp.len + nw - 1) / nw, cap);   // blocks the busiest wave of the team walks
                    }
                }
                if (cls != want) continue;
                if (gp.sliced) {
                    meta[g] = make_int4(pos, -1, -1, gp.parts);
                    pos += gp.parts;
                    continue;
                }
                int first = -1;
                for (int p = 0; p < gp.parts; ++p) {
                    int plen = piece_lo(gp.len, p + 1, gp.parts) - piece_lo(gp.len, p, gp.parts);
                    int nw = waves_of_part(plen, cap, waves);
                    int in_wg = pos % waves;
                    if (in_wg + nw > waves) pos += waves - in_wg;
                    if (p == 0) first = pos;
                    pos += nw;
                }
                const bool split = gp.parts > 1;
                meta[g] = make_int4(first, split ? tile_slots : -1, split ? split_groups : -1, gp.parts);
                if (split) { tile_slots += gp.parts; split_groups += 1; }
            }
        }
        int n_wgs = (pos + waves - 1) / waves;
        total_slots = n_wgs * waves;
        counts_out[0] = total_slots <= slot_capacity ? n_wgs : -1;   // -1: the table is too small, nothing usable
        counts_out[1] = tile_slots;
        counts_out[2] = split_groups;
        counts_out[3] = pos;
    }
    __syncthreads();
    const int n_slots = total_slots < slot_capacity ? total_slots : slot_capacity;
    for (int s = tid; s < n_slots; s += LB_THREADS) slots[s] = make_int4(-1, 0, 0, 0);
    __syncthreads();
    for (int g = tid; g < groups; g += LB_THREADS) {
        const int lo = offsets[g];
        const GroupPlan gp = plan_group(offsets[g + 1] - lo, cap, waves, allow_split, slice_max, slices);
        int pos = meta[g].x;
        if (gp.sliced) {
            for (int t = 0; t < gp.parts; ++t)
                if (pos + t < slot_capacity)
                    slots[pos + t] = make_int4(g, lo, lo + gp.len, sched_team_word((pos + t) % waves, 1, t, gp.parts));
            continue;
        }
        for (int p = 0; p < gp.parts; ++p) {
            const int pb = piece_lo(gp.len, p, gp.parts), pe = piece_lo(gp.len, p + 1, gp.parts);
            const int plen = pe - pb;
            const int nw = waves_of_part(plen, cap, waves);
            const int in_wg = pos % waves;
            if (in_wg + nw > waves) pos += waves - in_wg;
            for (int t = 0; t < nw; ++t) {
                const int b = lo + pb + piece_lo(plen, t, nw), e = lo + pb + piece_lo(plen, t + 1, nw);
                if (pos + t < slot_capacity)
                    slots[pos + t] = make_int4(g, b, e, sched_team_word(pos % waves, nw, p, gp.parts));
            }
            pos += nw;
        }
    }
}

// ---- launchers ------------------------------------------------------------

hipError_t launch_layout_build(const uint8_t *mask, int R, int C, int32_t *row_blocks,
                               int32_t *row_off, int32_t *col_blocks, int32_t *col_off,
                               int32_t *nnz_out, void *workspace, hipStream_t stream)
{
    layout_build_kernel<<<1, LB_THREADS, 0, stream>>>(mask, R, C, (int2 *)row_blocks, row_off,
                                                     (int2 *)col_blocks, col_off, nnz_out,
                                                     (int *)workspace);
    return hipGetLastError();
}

hipError_t launch_schedule_build(const int32_t *offsets, int groups, int cap, int waves,
                                 int flags, int slice_max, int slices, int32_t *sched, int64_t capacity,
                                 int32_t *counts_out, hipStream_t stream)
{
    schedule_build_kernel<<<1, LB_THREADS, 0, stream>>>(offsets, groups, cap, waves, flags, slice_max, slices,
                                                       (int4 *)sched, (int)(capacity - groups),
                                                       counts_out);
    return hipGetLastError();
}

}  // namespace bsa
