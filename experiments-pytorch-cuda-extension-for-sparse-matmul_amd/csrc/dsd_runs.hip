// DSD over RUNS of block rows: c = dense0(a) b for a row table, b stored [K][N] (the P V product of
// attention), fp16 / bf16, with the dense strips of a run resident in LDS.
//
// Why: in the walk of dsd_rows_f16_kernel every block brings its own 4 KB strip of b out of L2 next to
// its 2 KB from HBM, and a compute unit hands loads back in the order it took them, whichever wave
// they belong to: under a saturated HBM the strips, L2 hits all of them, arrive no sooner than the
// blocks queued in front of them.  Neighbouring rows of an attention mask share most of their columns
// (the strided / global ones all of them, the local window all but one), so a workgroup that owns a RUN
// of consecutive rows needs few distinct strips: it fetches each once into LDS (up to 39 x 4 KB of the
// 160 KB a gfx950 compute unit has) and its waves then read nothing but blocks from memory.
//
// A run is one workgroup; runs are cut so that they hold about the same number of pairs (the host picks
// the target so that one launch fills the compute units a whole number of times; a workgroup this size
// has a compute unit to itself).  The waves of a run share its pairs evenly, wherever the row boundaries
// fall: a row that is finished inside a wave's chunk is stored from there, a row that straddles waves is
// summed through LDS mailboxes by the wave in which it begins.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "../../include/bsa.h"
#include "bsa_device.hpp"
#include "bsa_internal.hpp"
#include "lds_tiles.hpp"
#include "group_walk.hpp"

namespace bsa {

// ---- the run schedule -----------------------------------------------------------------------------
// [RunRecord x capacity rows][one byte per pair].  The byte of a pair: bits 0-5 the LDS slot of its
// column's strip within its run, bit 7 set on the first pair of a row.
struct RunRecord {
    int row0, row1;       // block rows [row0, row1)
    int p0, p1;           // their pairs in the row table
    int n_cols;           // distinct block columns = strips the run keeps in LDS
    int table_rows;       // the table the schedule was cut from: its groups ...
    int table_nnz;        // ... and pairs (the walk leaves without a result when they are not its own)
    int pad;
    unsigned short cols[64];   // the first n_cols: block column of slot s; the rest repeat the last one
};
static_assert(sizeof(RunRecord) == RUN_RECORD_BYTES, "the host sizes the schedule with RUN_RECORD_BYTES");
static_assert(RUN_MAX_STRIPS * 4096 + 64 <= 163840 && RUN_MAX_STRIPS < 64, "strips and flags fit the LDS of one compute unit");

// One wavefront walks the rows in order.  Lane j looks at pair j of the row: is its column already in the
// run's list (kept in LDS), or new?  The row joins the run unless that would overflow the strips or
// overshoot the balanced target by more than stopping short undershoots it.
__global__ __launch_bounds__(64) void run_schedule_build_kernel(
    const BlockDesc *__restrict__ blocks, const int *__restrict__ offsets, int rows, int nnz, int target,
    int max_strips, RunRecord *__restrict__ runs, unsigned char *__restrict__ pair_byte, int *__restrict__ counts_out)
{
    __shared__ int cur[64];
    const int l = lane_id();
    const long long n_est = nnz > 0 ? (nnz + target - 1) / target : 1;     // runs the table would make at `target`
    int n_runs = 0, widest = 0, longest = 0, strips = 0, eligible = 1;
    int run_row0 = 0, run_p0 = 0, n_cur = 0;
    auto close_run = [&](int row1, int p1) {
        RunRecord *r = runs + n_runs;
        if (l == 0) {
            r->row0 = run_row0;
            r->row1 = row1;
            r->p0 = run_p0;
            r->p1 = p1;
            r->n_cols = n_cur;
            r->table_rows = rows;
            r->table_nnz = nnz;
            r->pad = 0;
        }
        r->cols[l] = (unsigned short)(n_cur > 0 ? cur[l < n_cur ? l : n_cur - 1] : 0);
        widest = n_cur > widest ? n_cur : widest;
        strips += n_cur;
        longest = p1 - run_p0 > longest ? p1 - run_p0 : longest;
        ++n_runs;
    };
    for (int r = 0; r < rows; ++r) {
        const int lo = offsets[r], n_r = offsets[r + 1] - lo;
        if (n_r > max_strips || n_r > 64) {      // a single row needs more strips than LDS holds
            eligible = 0;
            break;
        }
        const bool mine = l < n_r;
        const int col = mine ? blocks[lo + l].col() : -1;
        auto find = [&]() {
            int f = -1;
            for (int s = 0; s < n_cur; ++s) f = cur[s] == col ? s : f;
            return mine ? f : 0;
        };
        int found = find();
        unsigned long long fresh = __ballot(mine && found < 0);
        int n_new = __popcll(fresh);
        if (r > run_row0) {
            const long long cum = lo - run_p0;
            const bool overflow = n_cur + n_new > max_strips;
            const bool overshoot = (2 * cum + n_r) * n_est > 2ll * nnz;      // |cum + n_r - T| > |T - cum|, T = nnz / n_est
            if (overflow || overshoot) {
                close_run(r, lo);
                __syncthreads();
                run_row0 = r;
                run_p0 = lo;
                n_cur = 0;
                found = mine ? -1 : 0;
                fresh = __ballot(mine);
                n_new = n_r;
            }
        }
        int slot = found;
        if (mine && found < 0) {
            slot = n_cur + __popcll(fresh & ((1ull << l) - 1ull));
            cur[slot] = col;
        }
        if (mine) pair_byte[lo + l] = (unsigned char)(slot | (l == 0 ? 0x80 : 0));
        n_cur += n_new;
        __syncthreads();
    }
    if (eligible) close_run(rows, offsets[rows]);
    if (l == 0) {
        counts_out[0] = eligible ? n_runs : 0;
        counts_out[1] = widest;
        counts_out[2] = eligible ? strips : 0;
        counts_out[3] = longest;
    }
}

hipError_t launch_run_schedule_build(const int32_t *row_blocks, const int32_t *row_offsets, int rows, int nnz,
                                     int target_pairs, int max_strips, void *sched, int32_t *counts_out, hipStream_t st)
{
    RunRecord *runs = reinterpret_cast<RunRecord *>(sched);
    unsigned char *pair_byte = reinterpret_cast<unsigned char *>(sched) + (size_t)rows * sizeof(RunRecord);
    run_schedule_build_kernel<<<1, 64, 0, st>>>(reinterpret_cast<const BlockDesc *>(row_blocks), row_offsets, rows, nnz,
                                                target_pairs, max_strips, runs, pair_byte, counts_out);
    return hipGetLastError();
}

// ---- the walk ---------------------------------------------------------------------------------------
#ifndef BSA_RUN_DEPTH
#define BSA_RUN_DEPTH 3
#endif
constexpr int RUN_DEPTH = BSA_RUN_DEPTH;      // blocks in flight per wave

__device__ __forceinline__ void mailbox_put(const f4v (&acc)[8], float *box)
{
    const int l = lane_id();
#pragma unroll
    for (int t = 0; t < 8; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) box[(t * 4 + v) * WAVE + l] = acc[t][v];
}
__device__ __forceinline__ void mailbox_add(f4v (&acc)[8], const float *box)
{
    const int l = lane_id();
#pragma unroll
    for (int t = 0; t < 8; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[t][v] += box[(t * 4 + v) * WAVE + l];
}

// LDS: [strip slots, 4 KB each][mailboxes, 8 KB per wave: behind the strips when box_off != 0, else in their
// place once they are dead][one int per wave at info_off].  Operand layouts and accumulator meaning as in
// dsd_rows_f16_kernel.  sp and dn carry no __restrict__ on purpose: the order of the first requests below is
// part of the design and the compiler may not move them across the barriers.
template <bool BF, int MAXW>
__global__ __launch_bounds__(64 * MAXW) void dsd_runs_f16_kernel(
    const half_t *sp, const half_t *dn, half_t *__restrict__ out,
    const BlockDesc *__restrict__ blocks, const int *__restrict__ offsets,
    const RunRecord *__restrict__ runs, const unsigned char *__restrict__ pair_byte,
    int n_runs, int batches, int nnz, int DN, int KT, int XT, int sp_shared, int info_off, int box_off, int strips)
{
    extern __shared__ __align__(16) unsigned char lds_raw[];
    int batch, ri;
    if (!map_workgroup(n_runs, batches, batch, ri)) return;   // whole workgroup leaves together
    const int w = wave_id(), l = lane_id();
    const int W = (int)(blockDim.x >> 6);
    const RunRecord *rec = runs + ri;
    // the columns of the run: one vector load, issued together with the scalar loads of the record
    const int my_col = (int)rec->cols[l];
    const int row0 = rec->row0, row1 = rec->row1, p0 = rec->p0, p1 = rec->p1, n_cols = rec->n_cols;
    const int n = p1 - p0;
    // A schedule of another table, or a launch sized for another schedule (fewer LDS slots or waves than this run
    // needs), would index LDS and the operands out of range: the workgroup leaves instead, its rows unwritten.
    if (rec->table_rows * BS != XT || rec->table_nnz != nnz || n_cols > strips || n_cols < 0 || n < 0 || n > 64 * W ||
        row0 < 0 || row1 > rec->table_rows || p0 < 0 || p1 > nnz)
        return;
    int *info = reinterpret_cast<int *>(lds_raw + info_off);
    const int y0 = 64 * (int)blockIdx.y;
    const int g = l >> 4, i = l & 15;
    half_t *ob = out + (size_t)batch * XT * DN + y0 + 8 * g;

    if (n > 0) {
        const int b = p0 + (int)(((long long)n * w) / W), e = p0 + (int)(((long long)n * (w + 1)) / W);
        const half_t *spb = sp + (sp_shared ? 0 : (size_t)batch * nnz * BS2) + i * BS + 8 * g;
        const half_t *dnb = dn + (size_t)batch * DN * KT + y0;

        // ---- first requests: the strips (ceil(n_cols / W) per wave; the last round repeats the last strip
        // where a wave has none), the chunk's descriptors, the first blocks.  Every request is unconditional,
        // so the wait for the strips is exact and leaves the blocks in flight across the barrier. ----
        const int last = e > b ? e - 1 : p0;      // a valid pair for the requests of an idle wave
        int wt = b + l;
        wt = wt < e ? wt : last;
        int win_pos, win_byte;
        uint4 blk[RUN_DEPTH][2];
        // Pair p of a row table names block p.  Past the end of the chunk the request stays (the wait counts the
        // compiler derives stay exact) but every lane asks for the same 16 bytes of the run's record: one cache line
        // instead of a block, never used.
        const half_t *idle = reinterpret_cast<const half_t *>(rec);
        auto issue_block = [&](int p, uint4 (&bb)[2]) {
            const half_t *src = spb + (size_t)p * BS2;
            bb[0] = ldg16_stream(p < e ? src : idle);
            bb[1] = ldg16_stream(p < e ? src + 16 * BS : idle);
        };
        auto first_requests = [&](auto rounds_c) {
            constexpr int K = decltype(rounds_c)::value;
            uint4 st[K][4];
#pragma unroll
            for (int k = 0; k < K; ++k) {
                int s = w + k * W;
                s = s < n_cols ? s : n_cols - 1;
                const half_t *src = dnb + (size_t)(BS * __builtin_amdgcn_readlane(my_col, s)) * DN;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int c = l + 64 * q;
                    st[k][q] = ldg16(src + (size_t)(c >> 3) * DN + 8 * (c & 7));
                }
            }
            // no wave asks for a block (HBM) before every wave of the workgroup has asked for its strips (L2)
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            win_pos = blocks[wt].pos;
            win_byte = (int)pair_byte[wt];
#pragma unroll
            for (int d = 0; d < RUN_DEPTH; ++d) issue_block(b + d, blk[d]);
            asm volatile("" ::: "memory");      // the requests above do not sink below this point
#pragma unroll
            for (int k = 0; k < K; ++k)
#pragma unroll
                for (int q = 0; q < 4; ++q)     // the strips are needed here, the blocks are not
                    asm volatile("" : "+v"(st[k][q].x), "+v"(st[k][q].y), "+v"(st[k][q].z), "+v"(st[k][q].w));
#pragma unroll
            for (int k = 0; k < K; ++k) {
                const int s = w + k * W;
                if (s < n_cols) {
                    unsigned char *tile = lds_raw + (size_t)s * 4096;
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        // rows 8-15 and 24-31 (q odd) are stored with the halves of every piece exchanged
                        const uint4 v = (q & 1) ? make_uint4(st[k][q].z, st[k][q].w, st[k][q].x, st[k][q].y) : st[k][q];
                        *reinterpret_cast<uint4 *>(tile + put_strip16_addr(l, q)) = v;
                    }
                }
            }
        };
        const int rounds = (n_cols + W - 1) / W;
        if (rounds <= 1) first_requests(std::integral_constant<int, 1>{});
        else if (rounds == 2) first_requests(std::integral_constant<int, 2>{});
        else if (rounds == 3) first_requests(std::integral_constant<int, 3>{});
        else first_requests(std::integral_constant<int, 4>{});
        // what the owner of a row has to know about the waves behind it: bit 0 the wave holds pairs, bit 1 its
        // first pair goes on a row begun earlier (or it holds none: the row may go on behind it), bit 2 a row
        // begins inside its chunk
        const bool head = b < e && !((__builtin_amdgcn_readlane(win_byte, 0) >> 7) & 1);
        {
            const unsigned long long starts = __ballot(b + l < e && ((win_byte >> 7) & 1));
            if (l == 0) info[w] = (b < e ? 1 : 0) | (head || b >= e ? 2 : 0) | (starts != 0ull ? 4 : 0);
        }
        lds_barrier();

        // ---- the walk ----
        f4v acc[8] = {{0}, {0}, {0}, {0}, {0}, {0}, {0}, {0}};
        f4v acc_head[8];          // the end of a row begun in an earlier wave, kept until that wave can take it
        bool have_head = false;
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
        int cur = (int)((unsigned)__builtin_amdgcn_readlane(win_pos, 0) >> 16);
        bool first_group = true;
        // one block: its strip out of LDS, eight 16 x 16 x 32 products, then the request for the block
        // RUN_DEPTH further on
        auto step = [&](int p, uint4 (&bb)[2]) {
            if (p < e) {
                const int gp = (int)((unsigned)__builtin_amdgcn_readlane(win_pos, p - b) >> 16);
                const int slot = __builtin_amdgcn_readlane(win_byte, p - b) & 63;
                if (gp != cur) {
                    if (first_group && head) {
#pragma unroll
                        for (int t = 0; t < 8; ++t) acc_head[t] = acc[t];
                        have_head = true;
                    } else {
                        store_group(cur);
                    }
#pragma unroll
                    for (int t = 0; t < 8; ++t) acc[t] = f4v{0};
                    cur = gp;
                    first_group = false;
                }
                const unsigned char *tile = lds_raw + (size_t)slot * 4096;
                h8 dop[4];
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    h4 lo = lds_read_tr16(reinterpret_cast<const half_t *>(tile + get_strip16_addr(l, t, 0)));
                    h4 hi = lds_read_tr16(reinterpret_cast<const half_t *>(tile + get_strip16_addr(l, t, 1)));
                    dop[t] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                }
#pragma unroll
                for (int xh = 0; xh < 2; ++xh)
#pragma unroll
                    for (int t = 0; t < 4; ++t) acc[4 * xh + t] = mfma_16x16<BF>(dop[t], as_h8(bb[xh]), acc[4 * xh + t]);
            }
            issue_block(p + RUN_DEPTH, bb);
        };
        for (int p = b; p < e; p += RUN_DEPTH) {
#pragma unroll
            for (int d = 0; d < RUN_DEPTH; ++d) step(p + d, blk[d]);
        }

        // ---- rows that straddle waves ----
        const bool give = b < e && first_group && head;   // the whole chunk lies in a row an earlier wave owns
        if (box_off == 0) lds_barrier();                  // the strips are dead: their place holds the mailboxes now
        float *box = reinterpret_cast<float *>(lds_raw + box_off + (size_t)w * 8192);
        if (have_head) mailbox_put(acc_head, box);
        else if (give) mailbox_put(acc, box);
        lds_barrier();
        if (b < e && !give) {
            for (int v = w + 1; v < W; ++v) {
                const int iv = info[v];
                if (!(iv & 2)) break;
                if (iv & 1) mailbox_add(acc, reinterpret_cast<const float *>(lds_raw + box_off + (size_t)v * 8192));
                if (iv & 4) break;
            }
            store_group(cur);
        }
    }
    // rows without blocks: zeros
    for (int r = row0 + w; r < row1; r += W) {
        if (offsets[r + 1] == offsets[r]) {
#pragma unroll
            for (int xh = 0; xh < 2; ++xh) {
                half_t *orow = ob + (size_t)(BS * r + 16 * xh + i) * DN;
                stg16(orow, make_uint4(0, 0, 0, 0));
                stg16(orow + 32, make_uint4(0, 0, 0, 0));
            }
        }
    }
}

constexpr size_t RUN_LDS_MAX = 163840;     // what one workgroup may take on gfx950

template <class Kernel>
static hipError_t launch_runs(Kernel kernel, const RunsArgs &p, hipStream_t st)
{
    size_t lds = (size_t)p.strips * 4096;
    int box_off = 0;
    if (lds + (size_t)p.waves * 8192 + 64 <= RUN_LDS_MAX) {       // mailboxes of their own
        box_off = (int)lds;
        lds += (size_t)p.waves * 8192;
    } else if (lds < (size_t)p.waves * 8192) {
        lds = (size_t)p.waves * 8192;
    }
    const int info_off = (int)lds;
    lds += 64;
    if (lds > RUN_LDS_MAX) return hipErrorInvalidValue;
    hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (err != hipSuccess) return err;
    dim3 grid(8u * (unsigned)p.n_runs * (unsigned)((p.batches + 7) / 8), (unsigned)(p.N / 64)), block(64 * p.waves);
    const RunRecord *runs = reinterpret_cast<const RunRecord *>(p.sched);
    const unsigned char *pair_byte = reinterpret_cast<const unsigned char *>(p.sched) + (size_t)p.mask_rows * sizeof(RunRecord);
    kernel<<<grid, block, lds, st>>>((const half_t *)p.a, (const half_t *)p.b, (half_t *)p.c, (const BlockDesc *)p.blocks,
                                     p.offsets, runs, pair_byte, p.n_runs, p.batches, p.nnz, p.N, 32 * p.mask_cols,
                                     32 * p.mask_rows, p.sparse_shared ? 1 : 0, info_off, box_off, p.strips);
    return hipGetLastError();
}

hipError_t launch_dsd_runs(int dtype, const RunsArgs &p, hipStream_t st)
{
    static_assert(RUN_MAX_WAVES == 12, "the widest instantiation below");
    if (p.waves <= 8) {
        if (dtype == BSA_F16) return launch_runs(dsd_runs_f16_kernel<false, 8>, p, st);
        return launch_runs(dsd_runs_f16_kernel<true, 8>, p, st);
    }
    if (dtype == BSA_F16) return launch_runs(dsd_runs_f16_kernel<false, 12>, p, st);
    return launch_runs(dsd_runs_f16_kernel<true, 12>, p, st);
}

}  // namespace bsa
