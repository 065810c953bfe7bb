// Host-side launchers behind the C ABI (one per kernel family).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bsa {

hipError_t launch_layout_build(const uint8_t *mask, int R, int C, int32_t *row_blocks,
                               int32_t *row_off, int32_t *col_blocks, int32_t *col_off,
                               int32_t *nnz_out, void *workspace, hipStream_t stream);

hipError_t launch_schedule_build(const int32_t *offsets, int groups, int cap, int waves,
                                 int flags, int slice_max, int slices, int32_t *sched, int64_t capacity,
                                 int32_t *counts_out, hipStream_t stream);

hipError_t launch_to_sparse(int elem_size, const void *dense, void *sparse, const int32_t *row_blocks,
                            int nnz, int batches, int R, int C, hipStream_t stream);
hipError_t launch_to_dense(int elem_size, const void *sparse, void *dense, const uint8_t *mask,
                           const int32_t *ordinal_of, int nnz, int batches, int R, int C, hipStream_t stream);

struct MatmulArgs {
    const void *a, *b;
    void *c;
    const int32_t *blocks;
    const int32_t *sched;      // group records, then wavefront slots
    int groups;
    int sched_wgs, sched_waves;
    int tile_slots, split_groups;   // partial tiles / counters one (batch, strip) needs
    void *workspace;
    int nnz, batches;
    int M, N, K;
    bool tr_a, tr_b;
    bool sparse_shared;   // DSD / DDS: the sparse operand has no batch dimension
    bool row_table = false;   // DSD / DDS: `blocks` is the row-major table, whose pair p names block p
};

hipError_t launch_sdd(int dtype, const MatmulArgs &p, hipStream_t stream);
size_t gw_counter_bytes(int split_groups, int batches, int free_dim);
size_t gw_workspace_bytes(int tile_slots, int split_groups, int batches, int free_dim);
// group walk shared by DSD (dsd = true) and DDS
hipError_t launch_group_walk(int dtype, bool dsd, const MatmulArgs &p, hipStream_t stream);
// the same walk with the split-group workspace in the library's static device buffer (p.workspace is ignored)
hipError_t launch_group_walk_static_scratch(int dtype, bool dsd, const MatmulArgs &p, hipStream_t stream);

// DSD on a mask of 64 x 64 blocks (coarse tables: one pair per block)
struct Block64Args {
    const void *a, *b;
    void *c;
    const int32_t *blocks, *offsets;   // row table of the coarse mask
    const int32_t *sched;              // schedule of that table, built without splitting
    int coarse_rows, coarse_cols, coarse_nnz;
    int sched_wgs, sched_waves;
    int batches, N;
    bool sparse_shared;
};
hipError_t launch_dsd_block64(int dtype, const Block64Args &p, hipStream_t stream);

// DSD over runs of block rows with the dense strips of a run resident in LDS (dsd_runs.hip)
constexpr int RUN_RECORD_BYTES = 160;      // one record per run; the schedule is [records x mask rows][one byte per pair]
constexpr int RUN_MAX_STRIPS = 39;         // 4 KB each, next to the per-wave flags, in the 160 KB of a compute unit
constexpr int RUN_MAX_WAVES = 12;
hipError_t launch_run_schedule_build(const int32_t *row_blocks, const int32_t *row_offsets, int rows, int nnz,
                                     int target_pairs, int max_strips, void *sched, int32_t *counts_out,
                                     hipStream_t stream);
struct RunsArgs {
    const void *a, *b;
    void *c;
    const int32_t *blocks, *offsets;   // row table
    const void *sched;                 // run schedule of that table
    int n_runs, waves, strips;         // strips: the widest run's (counts_out[1] of the build)
    int mask_rows, mask_cols, nnz;
    int batches, N;
    bool sparse_shared;
};
hipError_t launch_dsd_runs(int dtype, const RunsArgs &p, hipStream_t stream);

struct SoftmaxArgs {
    const void *x;    // forward: scores; backward: y
    const void *dy;   // backward only
    void *out;
    const int32_t *blocks;
    const int32_t *sched;
    int groups;
    int sched_wgs, sched_waves;
    int nnz, batches;
    float scale;
    bool causal;
};

hipError_t launch_softmax_forward(int dtype, const SoftmaxArgs &p, hipStream_t stream);
hipError_t launch_softmax_backward(int dtype, const SoftmaxArgs &p, hipStream_t stream);

struct AttentionArgs {
    const void *q = nullptr, *k = nullptr, *v = nullptr;
    void *out = nullptr;            // forward: result; backward: the forward result (read)
    void *lse = nullptr;            // forward: optional output; backward: input
    const void *dout = nullptr;     // backward only
    void *p_out = nullptr, *ds_out = nullptr;   // row walk of the backward pass, both or neither: [batches, nnz, 32, 32]
    void *dq_out = nullptr;         // row walk, may be null: [batches, 32 mask_rows, head_dim]
    void *delta = nullptr;          // float [batches, 32 mask_rows], rowsum(dout o out): written by the row walk (may be
                                    // null there), read by the column walk
    void *dk_out = nullptr, *dv_out = nullptr;  // column walk: [batches, 32 mask_cols, head_dim]
    int nnz = 0;
    const int32_t *blocks = nullptr;
    const int32_t *sched = nullptr;
    int groups = 0;                 // block rows (block columns for the column walk)
    int sched_wgs = 0, sched_waves = 0;
    int tile_slots = 0, split_groups = 0;   // parked tiles / counters one batch entry needs for the split groups of this walk
    void *workspace = nullptr;
    int mask_rows = 0, mask_cols = 0, batches = 0;
    float scale = 1.f;
    bool causal = false;
    bool bf16 = false;      // operands are bfloat16, not fp16
    int head_dim = 64;      // 64 or 128
};

size_t attention_workspace_bytes(int tile_slots, int split_groups, int batches, int head_dim);
// row walk region first, then the column walk's; either may be empty
size_t attention_backward_workspace_bytes(int row_tile_slots, int row_split_groups, int col_tile_slots,
                                          int col_split_groups, int batches, int head_dim);
hipError_t launch_attention_forward(const AttentionArgs &p, hipStream_t stream);
hipError_t launch_attention_backward_scores(const AttentionArgs &p, hipStream_t stream);
hipError_t launch_attention_backward_dkdv(const AttentionArgs &p, hipStream_t stream);   // groups = block columns, head dim 64

}  // namespace bsa
