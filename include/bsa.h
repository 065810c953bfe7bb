/*
 * bsa.h - C ABI of libbsa_hip.so: block-sparse attention kernels for AMD
 * Instinct MI355X (gfx950), 32x32 blocks.
 *
 * This library takes the place of the reference's torch C++ extension
 * `sparse_ops` (pybind block sparse/native/sparse_kernels.cc:53-57, prototype
 * native/sparse_ops.h:10-14).  Every entry point takes raw device pointers,
 * plain sizes and a hipStream_t passed as void*; no torch types cross this
 * boundary.  All functions
 *   - return 0 on success and a negative BSA_ERR_* code otherwise,
 *   - never synchronise, never allocate and never touch the null stream
 *     unless the caller passes it,
 *   - validate their arguments on the host before any launch; a message for
 *     the last failure on the calling thread is kept for bsa_last_error().
 *
 * Table format (bit-exact with sparse/layout.py:21-36, decoded as in
 * sparse/native/sparse_layout.cuh:13-21 but with a 16-bit column):
 *   blocks   int32[2*nnz]  pairs (idx, (row << 16) + col); idx is the row-major
 *                          ordinal of the block and addresses the block inside
 *                          a sparse operand stored [batch, nnz, 32, 32]
 *   offsets  int32[G+1]    first pair of every group: G = mask rows for the
 *                          row layout, mask columns for the column layout
 * In the ROW layout pair p therefore has idx == p (the pairs are in row-major
 * order themselves); the softmax and the walks over a row layout rely on it and
 * address block p of a row without waiting for its pair.
 *
 * Schedule format (new in this build), int32[4] records:
 *   [0, groups)   one per group: (first slot, first partial-tile slot or -1,
 *                 ordinal among the split groups or -1, parts)
 *   then one per wavefront slot: (group, first pair, one-past-last pair, team),
 *                 team = first wave of the team inside its workgroup (bits 0-3)
 *                 | waves in the team (4-7) | part (8-19) | parts (20-31);
 *                 group = -1 marks an unused slot.
 * A workgroup owns `waves` consecutive slots.  A group longer than cap * waves
 * pairs is cut into parts; the waves of one part (a team) sit in one workgroup
 * and reduce through LDS, the parts of a group meet in a workspace.
 */
#ifndef BSA_H_
#define BSA_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BSA_BLOCK 32

enum bsa_dtype { BSA_F32 = 0, BSA_F16 = 1, BSA_BF16 = 2 };   /* bf16: fp32 accumulation, like fp16 */
enum bsa_mode { BSA_SDD = 0, BSA_DSD = 1, BSA_DDS = 2 };

enum bsa_status {
    BSA_OK = 0,
    BSA_ERR_INVALID = -1,   /* argument validation failed; nothing was launched */
    BSA_ERR_LAUNCH = -2,    /* the HIP runtime reported an error on launch      */
    BSA_ERR_UNSUPPORTED = -3
};

/* Library version, major * 10000 + minor * 100 + patch. */
int bsa_version(void);

/* Message of the last failure on this thread ("" if none). Never NULL. */
const char *bsa_last_error(void);

/* ---- layout tables ------------------------------------------------------
 * Device-side replacement of SparseLayout._create_layout (sparse/layout.py:14-38),
 * both orientations in one launch.
 *   mask         device uint8[R*C], row-major, nonzero = block present
 *   row_blocks   device int32[2*R*C] (capacity; the first 2*nnz are written)
 *   row_offsets  device int32[R+1]
 *   col_blocks   device int32[2*R*C]
 *   col_offsets  device int32[C+1]
 *   nnz_out      device int32[1]
 *   workspace    device, bsa_layout_workspace_bytes(R, C) bytes; afterwards it holds, as
 *                int32[R*C], for every cell the number of stored blocks in front of
 *                it in row-major order (the block index of a stored cell), which
 *                bsa_to_dense reads
 * Limits: 1 <= R <= 32767, 1 <= C <= 65535 (the packed position is 16+16 bit
 * in a signed int32).
 */
size_t bsa_layout_workspace_bytes(int mask_rows, int mask_cols);
int bsa_layout_build(const uint8_t *mask, int mask_rows, int mask_cols,
                     int32_t *row_blocks, int32_t *row_offsets,
                     int32_t *col_blocks, int32_t *col_offsets,
                     int32_t *nnz_out, void *workspace, void *stream);

/* ---- dense matrix <-> stack of its stored blocks ---------------------------
 * Replace SparseLayout.to_sparse / to_dense (sparse/layout.py:40-57).
 *   dense   [batches, 32 * mask_rows, 32 * mask_cols], contiguous
 *   sparse  [batches, nnz, 32, 32]
 *   bsa_to_sparse copies the stored blocks out of `dense` (row_blocks: the row table);
 *   bsa_to_dense writes every cell of `dense`: the stored blocks, zeros elsewhere
 *   (`mask` as given to bsa_layout_build, `ordinals` its workspace afterwards).
 * dtype: BSA_F32, BSA_F16 or BSA_BF16 (any 4- or 2-byte element type moves the same way).
 */
int bsa_to_sparse(int dtype, const void *dense, void *sparse, const int32_t *row_blocks,
                  int mask_rows, int mask_cols, int nnz, int batches, void *stream);
int bsa_to_dense(int dtype, const void *sparse, void *dense, const uint8_t *mask, const int32_t *ordinals,
                 int mask_rows, int mask_cols, int nnz, int batches, void *stream);

/* ---- wavefront schedule -------------------------------------------------
 * Splits every group of a table into chunks of about `cap` pairs, one chunk
 * per wavefront, and packs the wavefronts into workgroups of `waves`
 * wavefronts.  `flags`: with BSA_SCHED_SPLIT a group longer than cap * waves
 * pairs is cut into parts of at most that many pairs, which run in different
 * workgroups and meet in a workspace (DSD / DDS, the attention walks); without
 * it the group gets longer chunks (softmax: a row cannot be split across
 * workgroups).  With BSA_SCHED_LONGEST_FIRST long work is placed first instead
 * of in table order: split groups, then the unsplit ones by the length of their
 * longest chunk (quarters of cap), then the row-sliced ones by length (a
 * wavefront walks its chunk serially and a launch is only a round or two of
 * wavefronts, so the long rows at the end of a causal mask would otherwise start
 * last; it pays for the DSD / DDS walks and the softmax, not for the others).
 * Empty groups get one wavefront with an empty chunk (it writes the zeros).
 * With `slice_max` >= 0 (softmax only, at most 64) a group of at most slice_max
 * pairs is not chunked at all: it goes whole to `slices` wavefronts (2, 4 or 8;
 * `waves` must be a multiple), each taking 32 / slices of its 32 element rows
 * (team word: waves = 1, part = slice, parts = slices), and these wavefronts fill
 * workgroups of their own, at the front of the schedule (behind the other groups
 * with BSA_SCHED_LONGEST_FIRST).  The softmax kernels keep such a slice in
 * registers when the group has at most 48 (fp16 / bf16) or 24 (fp32) pairs and
 * slices is 4 in the forward kernel, and at most 24 pairs in the backward kernel
 * with slices 4 (fp16 / bf16) or 8 (fp32); other sliced groups are still computed
 * correctly, by a slower two-pass walk.  Pass slice_max = -1 for the matmul
 * schedules.
 * No counterpart in the reference, whose grids are (nnz, B) and
 * (B, M/32, N/32) (sparse/native/sparse_smm_gpu.cu:278-279).
 *   sched        device int32[4 * bsa_schedule_capacity(...)]
 *   counts_out   device int32[4]: workgroups the schedule uses (-1 if `capacity`
 *                was too small: the table is then unusable), partial-tile
 *                slots, split groups, wavefront slots in use
 */
int64_t bsa_schedule_capacity(int groups, int nnz, int cap, int waves);
enum bsa_sched_flags { BSA_SCHED_SPLIT = 1, BSA_SCHED_LONGEST_FIRST = 2 };
int bsa_schedule_build(const int32_t *offsets, int groups, int cap, int waves,
                       int flags, int slice_max, int slices, int32_t *sched,
                       int64_t capacity, int32_t *counts_out, void *stream);

/* ---- block-sparse matmul -----------------------------------------------
 * Replaces sparse_matmul's launch half: sparse_smm_32x32x32_kernel_wrapper and
 * sparse_hmm_32x32x32_kernel_wrapper (sparse/native/sparse_kernels.h:10-24,
 * sparse_smm_gpu.cu:270-293, sparse_hmm_gpu.cu:320-343).  The shape logic of
 * sparse_kernels.cc:12-37 stays with the caller, which passes the result:
 *   mode   BSA_SDD  c[b, idx]   = op(a)[b] (M x K) * op(b)[b] (K x N) on stored blocks
 *          BSA_DSD  c[b] (MxN)  = op(S(a))[b] * op(b)[b]
 *          BSA_DDS  c[b] (MxN)  = op(a)[b] * op(S(b))[b]
 *   op(x) = x or its transpose (tr_a / tr_b); dense operands are contiguous
 *   [batches, rows, cols] as stored, sparse ones [batches, nnz, 32, 32].
 *   blocks/offsets/sched must be those of the layout the reference's rule
 *   picks (sparse_kernels.cc:12): the ROW layout for sdd, for dsd without tr_a
 *   and for dds with tr_b; the COLUMN layout otherwise.  `groups` is that
 *   table's group count, `sched_wgs`/`sched_waves` describe its schedule.
 *   M, N, K are the dims of op(a) (M x K) and op(b) (K x N); every dim that
 *   runs along the sparse matrix must equal 32 * mask_rows / 32 * mask_cols
 *   (after the transpose), the free dense dim must be a multiple of 32.
 *   sched_tile_slots / sched_split_groups are counts_out[1] / [2] of the
 *   schedule.  DSD and DDS with split groups need a workspace of
 *   bsa_matmul_workspace_bytes(...) bytes that is ZERO before its first use;
 *   every launch leaves it zero again, so it can be reused by later launches
 *   on the same stream (launches that overlap in time need separate ones).
 *   SDD takes no workspace (null, 0).
 *   sparse_batches is `batches`, or 1 (DSD / DDS only) when ONE sparse operand [nnz, 32, 32] serves
 *   every batch entry (a block-sparse weight); the reference has no such case.
 * fp16 and bf16 accumulate in fp32.  Empty groups give zero rows / columns.
 */
size_t bsa_matmul_workspace_bytes(int mode, int sched_tile_slots, int sched_split_groups,
                                  int batches, int M, int N);
int bsa_matmul(int mode, int dtype, const void *a, const void *b, void *c,
               const int32_t *blocks, const int32_t *offsets, int groups,
               const int32_t *sched, int sched_wgs, int sched_waves,
               int sched_tile_slots, int sched_split_groups,
               void *workspace, size_t workspace_bytes,
               int mask_rows, int mask_cols, int nnz, int batches, int sparse_batches,
               int M, int N, int K, int tr_a, int tr_b, void *stream);

/* ---- block-sparse matmul for callers that cannot allocate -----------------
 * No counterpart in the reference.  For callers that cannot call hipMalloc or hand over a
 * workspace: code under HIP graph capture, tight serving loops, harnesses that forbid
 * allocation.  Same operation, arguments, checks and results as bsa_matmul (bit for bit: the
 * kernels are the same), but the partial tiles and counters of split groups live in a buffer
 * of BSA_STATIC_SCRATCH_BYTES that is part of the library's device code (one copy per GPU,
 * held until the process ends), so there is no workspace argument and the call allocates
 * nothing.  A schedule whose split groups need more than that is refused with
 * BSA_ERR_UNSUPPORTED (bsa_matmul_workspace_bytes() tells the need).  Every call clears the
 * counters it uses with a small kernel on `stream` before the walk, so the state a previous
 * call left behind does not matter.  All calls on one GPU share the buffer: calls that may
 * overlap in time on one GPU (different streams, different threads) race and must be
 * serialised by the caller.  The buffer used is that of the GPU the result `c` lives on,
 * whatever the caller's current device.  The first call on a GPU looks the buffer's address
 * up (hipGetSymbolAddress): make it outside graph capture.
 */
#define BSA_STATIC_SCRATCH_BYTES (16u << 20)
int bsa_matmul_noalloc(int mode, int dtype, const void *a, const void *b, void *c,
                       const int32_t *blocks, const int32_t *offsets, int groups,
                       const int32_t *sched, int sched_wgs, int sched_waves,
                       int sched_tile_slots, int sched_split_groups,
                       int mask_rows, int mask_cols, int nnz, int batches, int sparse_batches,
                       int M, int N, int K, int tr_a, int tr_b, void *stream);

/* ---- DSD on a mask of 64x64 blocks, the block as the unit of work -------------
 * No counterpart in the reference, whose kernels are 32x32x32 only (sparse/native/sparse_smm_gpu.cu:22,
 * :106, :192, and the hard-coded 32 of sparse/layout.py:42-45).  c[b] = S(a)[b] * b[b] for a sparse
 * operand whose mask is given in blocks of 64: a wavefront owns whole 64 x 64 blocks, so a dense strip
 * of 32 x 64 is fetched and staged once for the upper and the lower half of a block (half the strip
 * traffic of bsa_matmul on the same mask expanded to 32 x 32 tiles, same results).
 *   a        [sparse_batches, 4 * coarse_nnz, 32, 32]: the 2 x 2 tiles of every block, in the row-major
 *            order of the mask with every cell repeated twice along both axes (what bsa_layout_build /
 *            bsa_to_sparse give for that expanded mask); sparse_batches = batches, or 1 (shared)
 *   b        [batches, 64 * coarse_cols, N], c [batches, 64 * coarse_rows, N], N a multiple of 64
 *   coarse_row_blocks / coarse_row_offsets: the ROW table of the coarse mask (one pair per block)
 *   sched    schedule of that table from bsa_schedule_build WITHOUT BSA_SCHED_SPLIT and with at most
 *            4 waves per workgroup (a group never leaves its workgroup; no workspace is needed)
 * fp16 / bf16, no transposes; everything else goes through bsa_matmul on the expanded tables.
 */
int bsa_matmul_dsd_block64(int dtype, const void *a, const void *b, void *c,
                           const int32_t *coarse_row_blocks, const int32_t *coarse_row_offsets,
                           const int32_t *sched, int sched_wgs, int sched_waves,
                           int coarse_rows, int coarse_cols, int coarse_nnz, int batches, int sparse_batches,
                           int N, void *stream);

/* ---- DSD over runs of block rows, the dense strips of a run resident in LDS -----
 * No counterpart in the reference, whose DSD kernel reloads the dense tile of every block
 * (sparse/native/sparse_smm_gpu.cu:131-155).  c[b] = S(a)[b] * b[b] for the ROW table, no transposes,
 * fp16 / bf16, N a multiple of 64: the same product, on the same tables, as bsa_matmul(BSA_DSD).
 * A run is a range of consecutive block rows handled by one workgroup that has a compute unit to
 * itself: it fetches each distinct 32 x 64 strip of b that its rows name once into LDS (at most 39
 * strips) and then reads nothing but blocks from memory.  Pays when neighbouring rows share most of
 * their columns (local + strided / global attention masks); tables with a row of more than
 * max_strips blocks are not eligible.
 *   bsa_run_schedule_bytes   device bytes of the schedule of a table
 *   bsa_run_schedule_build   cuts the rows into runs of about target_pairs pairs (nearest row
 *                            boundary) and at most max_strips (1..39) distinct columns;
 *                            counts_out device int32[4]: runs (0: not eligible), strips of the
 *                            widest run, strips of all runs together (pairs / strips = how often a
 *                            fetched strip is used), pairs of the longest run
 *   bsa_matmul_dsd_runs      n_runs, run_strips, run_pairs: counts_out[0], [1], [3]; waves per
 *                            workgroup (1..12) with run_strips <= 4 waves and run_pairs <= 64 waves.
 *                            Results agree with bsa_matmul to the rounding of the fp32 sums (the
 *                            pairs of a row are summed in a different order).
 */
int64_t bsa_run_schedule_bytes(int mask_rows, int nnz);
int bsa_run_schedule_build(const int32_t *row_blocks, const int32_t *row_offsets, int mask_rows, int nnz,
                           int target_pairs, int max_strips, void *sched, int64_t sched_bytes,
                           int32_t *counts_out, void *stream);
int bsa_matmul_dsd_runs(int dtype, const void *a, const void *b, void *c,
                        const int32_t *row_blocks, const int32_t *row_offsets,
                        const void *run_sched, int n_runs, int run_strips, int run_pairs, int waves,
                        int mask_rows, int mask_cols, int nnz, int batches, int sparse_batches,
                        int N, void *stream);

/* ---- block-sparse softmax ----------------------------------------------
 * Replaces sparse_softmax_forward / sparse_softmax_backward
 * (sparse_softmax.cu:208-258) and their kernels (:113-205), with two additions:
 * the scores are multiplied by `scale` before the exponential, and with
 * `causal` != 0 every element whose global column exceeds its global row
 * counts as -inf.  x, y, dy, dx are [batches, nnz, 32, 32]; tables and schedule
 * are those of the ROW layout.  Rows with nothing unmasked yield zeros.
 *   forward : y  = softmax_row(scale * x)
 *   backward: dx = scale * (dy - sum_row(dy * y)) * y
 * Math is fp32 for every dtype.
 */
int bsa_softmax_forward(int dtype, const void *x, void *y,
                        const int32_t *row_blocks, const int32_t *row_offsets,
                        const int32_t *sched, int sched_wgs, int sched_waves,
                        int mask_rows, int mask_cols, int nnz, int batches,
                        float scale, int causal, void *stream);
int bsa_softmax_backward(int dtype, const void *y, const void *dy, void *dx,
                         const int32_t *row_blocks, const int32_t *row_offsets,
                         const int32_t *sched, int sched_wgs, int sched_waves,
                         int mask_rows, int mask_cols, int nnz, int batches,
                         float scale, void *stream);

/* ---- fused block-sparse attention, forward ----------------------------------
 * out = softmax_row(scale * q k^T restricted to the stored blocks, causal if asked) v in one launch:
 * the chain SDD -> softmax -> DSD that a caller of the reference writes with two calls of
 * sparse_matmul (sparse/matmul.py:57, kernels sparse_smm_gpu.cu:22-95 and :106-181) around the
 * softmax of sparse_softmax.cu:113-155, without the [batches, nnz, 32, 32] scores ever being
 * stored.  Same meaning as bsa_matmul(SDD, q, k, tr_b = 1), bsa_softmax_forward, bsa_matmul(DSD)
 * in a row; the probabilities are rounded to fp16 before the second product, as there.
 *   q    [batches, 32 * mask_rows, head_dim], k, v  [batches, 32 * mask_cols, head_dim], contiguous
 *   out  [batches, 32 * mask_rows, head_dim]; rows without stored (or unmasked) blocks give zeros
 *   lse  optional (may be NULL) float[batches, 32 * mask_rows]: log2 of every row's sum of
 *        2^(scale * log2(e) * score); +inf for a row that sees nothing.  The backward pass needs it.
 *   tables / schedule: those of the ROW layout, the schedule built with slice_max = -1.  With
 *   BSA_SCHED_SPLIT a block row longer than cap * waves is cut into parts that run in different
 *   workgroups and meet in `workspace` (sched_tile_slots, sched_split_groups: counts_out[1], [2] of
 *   bsa_schedule_build; bsa_attention_workspace_bytes() bytes, zeroed once by the caller: every launch
 *   leaves it zero again, so launches ordered on one stream may share it; NULL when nothing is split).
 * fp16 and bf16 only, head_dim 64 or 128 (BSA_ERR_UNSUPPORTED otherwise).
 */
size_t bsa_attention_workspace_bytes(int sched_tile_slots, int sched_split_groups, int batches, int head_dim);
int bsa_attention_forward(int dtype, const void *q, const void *k, const void *v, void *out, float *lse,
                          const int32_t *row_blocks, const int32_t *row_offsets,
                          const int32_t *sched, int sched_wgs, int sched_waves,
                          int sched_tile_slots, int sched_split_groups, void *workspace, size_t workspace_bytes,
                          int mask_rows, int mask_cols, int nnz, int batches, int head_dim,
                          float scale, int causal, void *stream);

/* The walk over the rows of the attention backward pass in one launch: from q, k, v, the gradient
 * `dout` of the result, the forward result `out` and `lse`, the probabilities and the score
 * gradients of every stored block, and the gradient of q,
 *   p_out  = softmax probabilities                         [batches, nnz, 32, 32]
 *   ds_out = scale * p o (dout v^T - rowsum(dout o out))   [batches, nnz, 32, 32]
 *   dq_out = ds k                                          [batches, 32 * mask_rows, head_dim]; may be NULL
 * i.e. what SDD(q, k), the softmax forward, SDD(dout, v), the softmax backward and DSD(ds, k) of the
 * unfused chain produce with five launches (sparse_smm_gpu.cu:22-95 twice, sparse_softmax.cu:113-205,
 * sparse_smm_gpu.cu:106-181).  The caller finishes with the two products that walk the columns,
 * dk = ds^T q and dv = p^T dout (bsa_matmul, mode 1, transposed first operand), and with
 * dq = ds k as a third one if it passed dq_out = NULL.
 * Same tables, schedule and limits as the forward; a schedule with split rows needs, when dq_out is
 * asked for, bsa_attention_backward_workspace_bytes(sched_tile_slots, sched_split_groups, 0, 0, ...) bytes
 * of workspace under the same rules (zeroed once, left zero).
 */
size_t bsa_attention_backward_workspace_bytes(int row_tile_slots, int row_split_groups, int col_tile_slots,
                                              int col_split_groups, int batches, int head_dim);
int bsa_attention_backward_scores(int dtype, const void *q, const void *k, const void *v, const void *dout,
                                  const void *out, const float *lse, void *p_out, void *ds_out, void *dq_out,
                                  const int32_t *row_blocks, const int32_t *row_offsets,
                                  const int32_t *sched, int sched_wgs, int sched_waves,
                                  int sched_tile_slots, int sched_split_groups, void *workspace, size_t workspace_bytes,
                                  int mask_rows, int mask_cols, int nnz, int batches, int head_dim,
                                  float scale, int causal, void *stream);

/* The whole backward pass of that operator in two launches, with no block stack in memory: a walk over
 * the rows that rebuilds the probabilities and the score gradients in registers and accumulates
 *   dq_out = ds k                       [batches, 32 * mask_rows, head_dim]
 * (and leaves rowsum(dout o out) in `delta_ws`, float [batches, 32 * mask_rows], caller-provided), and
 * a walk over the columns that rebuilds them a second time and accumulates
 *   dk_out = ds^T q,  dv_out = p^T dout [batches, 32 * mask_cols, head_dim].
 * Seven launches in the unfused chain (sparse/matmul.py:27-52 three times over, sparse_softmax.cu:165-205,233-258).
 * Row tables with a schedule built with slice_max = -1; column tables with a schedule of their own built the
 * same way on col_offsets.  Either schedule may split long groups (BSA_SCHED_SPLIT): their parts add up in
 * `workspace`, bsa_attention_backward_workspace_bytes(counts_out[1], [2] of the row schedule, of the column
 * schedule, ...) bytes, zeroed once by the caller and left zero by every launch; NULL when nothing is split.
 * fp16 / bf16, head_dim 64 only (BSA_ERR_UNSUPPORTED otherwise: use bsa_attention_backward_scores and two
 * bsa_matmul calls).
 */
int bsa_attention_backward(int dtype, const void *q, const void *k, const void *v, const void *dout,
                           const void *out, const float *lse, void *dq_out, void *dk_out, void *dv_out,
                           float *delta_ws,
                           const int32_t *row_blocks, const int32_t *row_offsets,
                           const int32_t *row_sched, int row_sched_wgs, int row_sched_waves,
                           int row_tile_slots, int row_split_groups,
                           const int32_t *col_blocks, const int32_t *col_offsets,
                           const int32_t *col_sched, int col_sched_wgs, int col_sched_waves,
                           int col_tile_slots, int col_split_groups,
                           void *workspace, size_t workspace_bytes,
                           int mask_rows, int mask_cols, int nnz, int batches, int head_dim,
                           float scale, int causal, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* BSA_H_ */
