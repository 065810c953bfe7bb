// C ABI of libbsa_hip.so: argument validation and dispatch (see include/bsa.h).
// Takes over what the reference does in sparse/native/sparse_kernels.cc:39-46
// (dtype switch) and in its kernel wrappers (sparse_smm_gpu.cu:270-293), and
// adds the checks the reference lacks: every size the kernels index with is
// validated on the host before a launch.
#include <cstdarg>
#include <cstdio>

#include "../../include/bsa.h"
#include "bsa_internal.hpp"

namespace {

thread_local char g_error[512] = "";

int fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(hipError_t err, const char *what)
{
    if (err == hipSuccess) return BSA_OK;
    return fail(BSA_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(err));
}

constexpr int MAX_WAVES = 8;
constexpr long long MAX_GRID = 2147483647LL;

int check_schedule(const int32_t *sched, int sched_wgs, int sched_waves, int batches, const char *who)
{
    if (!sched) return fail(BSA_ERR_INVALID, "%s: schedule is null", who);
    if (sched_waves < 1 || sched_waves > MAX_WAVES)
        return fail(BSA_ERR_INVALID, "%s: schedule waves per workgroup %d outside [1, %d]", who, sched_waves, MAX_WAVES);
    if (sched_wgs < 1) return fail(BSA_ERR_INVALID, "%s: schedule has %d workgroups", who, sched_wgs);
    if (8LL * sched_wgs * ((batches + 7) / 8) > MAX_GRID)
        return fail(BSA_ERR_INVALID, "%s: grid of %d workgroups x %d batches is too large", who, sched_wgs, batches);
    return BSA_OK;
}

}  // namespace

extern "C" {

int bsa_version(void) { return 100; }

const char *bsa_last_error(void) { return g_error; }

size_t bsa_layout_workspace_bytes(int mask_rows, int mask_cols)
{
    if (mask_rows < 1 || mask_cols < 1) return 0;
    return (size_t)mask_rows * (size_t)mask_cols * sizeof(int32_t);
}

int bsa_layout_build(const uint8_t *mask, int mask_rows, int mask_cols,
                     int32_t *row_blocks, int32_t *row_offsets,
                     int32_t *col_blocks, int32_t *col_offsets,
                     int32_t *nnz_out, void *workspace, void *stream)
{
    if (mask_rows < 1 || mask_rows > 32767 || mask_cols < 1 || mask_cols > 65535)
        return fail(BSA_ERR_INVALID, "bsa_layout_build: mask shape %d x %d outside [1, 32767] x [1, 65535]",
                    mask_rows, mask_cols);
    if ((long long)mask_rows * mask_cols > (1LL << 28))
        return fail(BSA_ERR_INVALID, "bsa_layout_build: mask of %d x %d cells is too large", mask_rows, mask_cols);
    if (!mask || !row_blocks || !row_offsets || !col_blocks || !col_offsets || !nnz_out || !workspace)
        return fail(BSA_ERR_INVALID, "bsa_layout_build: null pointer argument");
    return check_launch(bsa::launch_layout_build(mask, mask_rows, mask_cols, row_blocks, row_offsets,
                                                 col_blocks, col_offsets, nnz_out, workspace,
                                                 (hipStream_t)stream),
                        "bsa_layout_build");
}

static int check_block_copy(const char *who, int dtype, const void *a, const void *b, const void *t0, const void *t1,
                            int mask_rows, int mask_cols, int nnz, int batches)
{
    if (dtype != BSA_F32 && dtype != BSA_F16 && dtype != BSA_BF16)
        return fail(BSA_ERR_UNSUPPORTED, "%s: unsupported dtype %d (fp32 = 0, fp16 = 1, bf16 = 2)", who, dtype);
    if (mask_rows < 1 || mask_rows > 32767 || mask_cols < 1 || mask_cols > 65535)
        return fail(BSA_ERR_INVALID, "%s: mask shape %d x %d out of range", who, mask_rows, mask_cols);
    if (nnz < 0 || (long long)nnz > (long long)mask_rows * mask_cols)
        return fail(BSA_ERR_INVALID, "%s: nnz %d does not fit a %d x %d mask", who, nnz, mask_rows, mask_cols);
    if (batches < 1) return fail(BSA_ERR_INVALID, "%s: batches %d < 1", who, batches);
    if (!a || !t0 || !t1 || (!b && nnz > 0)) return fail(BSA_ERR_INVALID, "%s: null pointer argument", who);
    return BSA_OK;
}

int bsa_to_sparse(int dtype, const void *dense, void *sparse, const int32_t *row_blocks,
                  int mask_rows, int mask_cols, int nnz, int batches, void *stream)
{
    if (nnz == 0 && dense) return BSA_OK;
    int rc = check_block_copy("bsa_to_sparse", dtype, dense, sparse, row_blocks, row_blocks, mask_rows, mask_cols, nnz, batches);
    if (rc) return rc;
    return check_launch(bsa::launch_to_sparse(dtype == BSA_F32 ? 4 : 2, dense, sparse, row_blocks, nnz, batches,
                                              mask_rows, mask_cols, (hipStream_t)stream), "bsa_to_sparse");
}

int bsa_to_dense(int dtype, const void *sparse, void *dense, const uint8_t *mask, const int32_t *ordinals,
                 int mask_rows, int mask_cols, int nnz, int batches, void *stream)
{
    int rc = check_block_copy("bsa_to_dense", dtype, dense, sparse, mask, ordinals, mask_rows, mask_cols, nnz, batches);
    if (rc) return rc;
    if ((long long)mask_rows * mask_cols > (1LL << 31) - 8)
        return fail(BSA_ERR_INVALID, "bsa_to_dense: %d x %d cells do not fit the launch", mask_rows, mask_cols);
    return check_launch(bsa::launch_to_dense(dtype == BSA_F32 ? 4 : 2, sparse, dense, mask, ordinals, nnz, batches,
                                             mask_rows, mask_cols, (hipStream_t)stream), "bsa_to_dense");
}

int64_t bsa_schedule_capacity(int groups, int nnz, int cap, int waves)
{
    if (groups < 1 || nnz < 0 || cap < 1 || waves < 1) return 0;
    // waves: sum over parts of (len / cap + 1) <= nnz / cap + parts, parts <= nnz / (cap * waves) + groups;
    // first-fit padding wastes less than the waves it pads for
    int64_t slots = 2 * (2 * ((int64_t)nnz / cap) + groups + 1) + 2 * waves;
    slots += 6 * (int64_t)groups;   // row-sliced groups take up to 8 slots each
    return slots + groups;   // one record per group in front
}

int bsa_schedule_build(const int32_t *offsets, int groups, int cap, int waves, int flags, int slice_max,
                       int slices, int32_t *sched, int64_t capacity, int32_t *counts_out, void *stream)
{
    if (flags < 0 || flags > (BSA_SCHED_SPLIT | BSA_SCHED_LONGEST_FIRST))
        return fail(BSA_ERR_INVALID, "bsa_schedule_build: unknown flags %d", flags);
    if (slice_max < -1 || slice_max > 64)
        return fail(BSA_ERR_INVALID, "bsa_schedule_build: slice_max %d outside [-1, 64]", slice_max);
    if (slice_max >= 0 && slices != 2 && slices != 4 && slices != 8)
        return fail(BSA_ERR_INVALID, "bsa_schedule_build: slices must be 2, 4 or 8, got %d", slices);
    if (slice_max >= 0 && waves % slices != 0)
        return fail(BSA_ERR_INVALID, "bsa_schedule_build: %d waves per workgroup do not hold whole groups of %d slices",
                    waves, slices);
    if (!offsets || !sched || !counts_out) return fail(BSA_ERR_INVALID, "bsa_schedule_build: null pointer argument");
    if (groups < 1 || groups > 65535) return fail(BSA_ERR_INVALID, "bsa_schedule_build: %d groups outside [1, 65535]", groups);
    if (cap < 1) return fail(BSA_ERR_INVALID, "bsa_schedule_build: cap %d < 1", cap);
    if (waves < 1 || waves > MAX_WAVES)
        return fail(BSA_ERR_INVALID, "bsa_schedule_build: waves %d outside [1, %d]", waves, MAX_WAVES);
    if (capacity < 2 * ((int64_t)groups + 1) + waves + groups || capacity > (1LL << 28))
        return fail(BSA_ERR_INVALID, "bsa_schedule_build: capacity %lld too small for %d groups (use bsa_schedule_capacity)",
                    (long long)capacity, groups);
    return check_launch(bsa::launch_schedule_build(offsets, groups, cap, waves, flags, slice_max, slices, sched, capacity,
                                                   counts_out, (hipStream_t)stream),
                        "bsa_schedule_build");
}

size_t bsa_matmul_workspace_bytes(int mode, int sched_tile_slots, int sched_split_groups,
                                  int batches, int M, int N)
{
    if (mode == BSA_SDD || sched_tile_slots <= 0 || sched_split_groups <= 0 || batches < 1) return 0;
    return bsa::gw_workspace_bytes(sched_tile_slots, sched_split_groups, batches, mode == BSA_DSD ? N : M);
}

static int matmul_checked(const char *who, bool static_scratch, int mode, int dtype, const void *a, const void *b, void *c,
                          const int32_t *blocks, const int32_t *offsets, int groups,
                          const int32_t *sched, int sched_wgs, int sched_waves,
                          int sched_tile_slots, int sched_split_groups,
                          void *workspace, size_t workspace_bytes,
                          int mask_rows, int mask_cols, int nnz, int batches, int sparse_batches,
                          int M, int N, int K, int tr_a, int tr_b, void *stream)
{
    if (mode != BSA_SDD && mode != BSA_DSD && mode != BSA_DDS)
        return fail(BSA_ERR_INVALID, "%s: unknown mode %d", who, mode);
    if (dtype != BSA_F32 && dtype != BSA_F16 && dtype != BSA_BF16)
        return fail(BSA_ERR_UNSUPPORTED, "%s: unsupported dtype %d (fp32 = 0, fp16 = 1, bf16 = 2)", who, dtype);
    // with nnz == 0 the table and the sparse tensor are empty and may be null
    const bool a_needed = nnz > 0 || mode != BSA_DSD, b_needed = nnz > 0 || mode != BSA_DDS;
    const bool c_needed = nnz > 0 || mode != BSA_SDD;
    if ((!a && a_needed) || (!b && b_needed) || (!c && c_needed) || (!blocks && nnz > 0) || !offsets)
        return fail(BSA_ERR_INVALID, "%s: null pointer argument", who);
    if (mask_rows < 1 || mask_rows > 32767 || mask_cols < 1 || mask_cols > 65535)
        return fail(BSA_ERR_INVALID, "%s: mask shape %d x %d out of range", who, mask_rows, mask_cols);
    if (nnz < 0 || (long long)nnz > (long long)mask_rows * mask_cols)
        return fail(BSA_ERR_INVALID, "%s: nnz %d does not fit a %d x %d mask", who, nnz, mask_rows, mask_cols);
    if (batches < 1) return fail(BSA_ERR_INVALID, "%s: batches %d < 1", who, batches);
    if (sparse_batches != batches && (sparse_batches != 1 || mode == BSA_SDD))
        return fail(BSA_ERR_INVALID, "%s: sparse_batches must equal batches (%d), or be 1 for dsd / dds; got %d", who,
                    batches, sparse_batches);
    if (M < 1 || N < 1 || K < 1 || M % BSA_BLOCK || N % BSA_BLOCK || K % BSA_BLOCK)
        return fail(BSA_ERR_INVALID, "%s: M, N, K = %d, %d, %d must be positive multiples of %d", who, M, N, K, BSA_BLOCK);
    int rc = check_schedule(sched, sched_wgs, sched_waves, batches, who);
    if (rc) return rc;

    // which table the caller must have passed, and what the sparse matrix spans
    const bool row_table = mode == BSA_SDD || (mode == BSA_DSD && !tr_a) || (mode == BSA_DDS && tr_b);
    const int want_groups = row_table ? mask_rows : mask_cols;
    if (groups != want_groups)
        return fail(BSA_ERR_INVALID, "%s: table has %d groups, the %s layout of a %d x %d mask has %d", who,
                    groups, row_table ? "row" : "column", mask_rows, mask_cols, want_groups);
    const int SR = BSA_BLOCK * mask_rows, SC = BSA_BLOCK * mask_cols;
    if (mode == BSA_SDD) {
        if (M != SR || N != SC)
            return fail(BSA_ERR_INVALID, "%s sdd: op(a) has %d rows and op(b) %d columns, the layout spans %d x %d", who,
                        M, N, SR, SC);
    } else if (mode == BSA_DSD) {
        const int m_want = tr_a ? SC : SR, k_want = tr_a ? SR : SC;
        if (M != m_want || K != k_want)
            return fail(BSA_ERR_INVALID, "%s dsd: M, K = %d, %d but op(sparse a) is %d x %d", who, M, K, m_want, k_want);
    } else {
        const int k_want = tr_b ? SC : SR, n_want = tr_b ? SR : SC;
        if (K != k_want || N != n_want)
            return fail(BSA_ERR_INVALID, "%s dds: K, N = %d, %d but op(sparse b) is %d x %d", who, K, N, k_want, n_want);
    }
    const int free_dim = mode == BSA_SDD ? K : (mode == BSA_DSD ? N : M);
    if ((free_dim + 63) / 64 > 65535)
        return fail(BSA_ERR_INVALID, "%s: dense dimension %d is too large", who, free_dim);

    if (sched_tile_slots < 0 || sched_split_groups < 0 || (sched_tile_slots > 0) != (sched_split_groups > 0))
        return fail(BSA_ERR_INVALID, "%s: schedule split counts %d, %d are inconsistent", who,
                    sched_tile_slots, sched_split_groups);
    const size_t ws_need = bsa_matmul_workspace_bytes(mode, sched_tile_slots, sched_split_groups, batches, M, N);
    if (static_scratch) {
        if (ws_need > (size_t)BSA_STATIC_SCRATCH_BYTES)
            return fail(BSA_ERR_UNSUPPORTED, "%s: the split groups of this schedule need %zu bytes of scratch, the "
                        "library's static buffer holds %zu (use bsa_matmul with a workspace of the caller's)", who,
                        ws_need, (size_t)BSA_STATIC_SCRATCH_BYTES);
    } else if (ws_need > 0 && (!workspace || workspace_bytes < ws_need)) {
        return fail(BSA_ERR_INVALID, "%s: workspace of %zu bytes needed, %zu given", who, ws_need, workspace_bytes);
    }

    bsa::MatmulArgs p{a, b, c, blocks, sched, groups, sched_wgs, sched_waves, sched_tile_slots, sched_split_groups,
                      workspace, nnz, batches, M, N, K, tr_a != 0, tr_b != 0, sparse_batches != batches};
    p.row_table = row_table;
    if (nnz == 0 && mode == BSA_SDD) return BSA_OK;   // nothing to write
    hipError_t err;
    if (mode == BSA_SDD) err = bsa::launch_sdd(dtype, p, (hipStream_t)stream);
    else if (static_scratch) err = bsa::launch_group_walk_static_scratch(dtype, mode == BSA_DSD, p, (hipStream_t)stream);
    else err = bsa::launch_group_walk(dtype, mode == BSA_DSD, p, (hipStream_t)stream);
    return check_launch(err, who);
}

int bsa_matmul(int mode, int dtype, const void *a, const void *b, void *c,
               const int32_t *blocks, const int32_t *offsets, int groups,
               const int32_t *sched, int sched_wgs, int sched_waves,
               int sched_tile_slots, int sched_split_groups,
               void *workspace, size_t workspace_bytes,
               int mask_rows, int mask_cols, int nnz, int batches, int sparse_batches,
               int M, int N, int K, int tr_a, int tr_b, void *stream)
{
    return matmul_checked("bsa_matmul", false, mode, dtype, a, b, c, blocks, offsets, groups, sched, sched_wgs,
                          sched_waves, sched_tile_slots, sched_split_groups, workspace, workspace_bytes, mask_rows,
                          mask_cols, nnz, batches, sparse_batches, M, N, K, tr_a, tr_b, stream);
}

int bsa_matmul_noalloc(int mode, int dtype, const void *a, const void *b, void *c,
                       const int32_t *blocks, const int32_t *offsets, int groups,
                       const int32_t *sched, int sched_wgs, int sched_waves,
                       int sched_tile_slots, int sched_split_groups,
                       int mask_rows, int mask_cols, int nnz, int batches, int sparse_batches,
                       int M, int N, int K, int tr_a, int tr_b, void *stream)
{
    return matmul_checked("bsa_matmul_noalloc", true, mode, dtype, a, b, c, blocks, offsets, groups, sched, sched_wgs,
                          sched_waves, sched_tile_slots, sched_split_groups, nullptr, 0, mask_rows, mask_cols, nnz,
                          batches, sparse_batches, M, N, K, tr_a, tr_b, stream);
}


int bsa_matmul_dsd_block64(int dtype, const void *a, const void *b, void *c,
                           const int32_t *coarse_row_blocks, const int32_t *coarse_row_offsets,
                           const int32_t *sched, int sched_wgs, int sched_waves,
                           int coarse_rows, int coarse_cols, int coarse_nnz, int batches, int sparse_batches,
                           int N, void *stream)
{
    const char *who = "bsa_matmul_dsd_block64";
    if (dtype != BSA_F16 && dtype != BSA_BF16)
        return fail(BSA_ERR_UNSUPPORTED, "%s: fp16 (dtype 1) and bf16 (dtype 2) are built, got %d", who, dtype);
    if (coarse_rows < 1 || coarse_rows > 16383 || coarse_cols < 1 || coarse_cols > 32767)
        return fail(BSA_ERR_INVALID, "%s: mask of %d x %d blocks of 64 out of range", who, coarse_rows, coarse_cols);
    if (coarse_nnz < 0 || (long long)coarse_nnz > (long long)coarse_rows * coarse_cols)
        return fail(BSA_ERR_INVALID, "%s: %d blocks do not fit a %d x %d mask", who, coarse_nnz, coarse_rows, coarse_cols);
    if ((long long)coarse_nnz * 4 > 2147483647LL / 2)
        return fail(BSA_ERR_INVALID, "%s: too many blocks (%d)", who, coarse_nnz);
    if (batches < 1 || (sparse_batches != batches && sparse_batches != 1))
        return fail(BSA_ERR_INVALID, "%s: batches %d, sparse_batches %d", who, batches, sparse_batches);
    if (N < 64 || N % 64)
        return fail(BSA_ERR_UNSUPPORTED, "%s: the dense width must be a positive multiple of 64, got %d (use bsa_matmul "
                    "on the expanded tables)", who, N);
    if (N / 64 > 65535) return fail(BSA_ERR_INVALID, "%s: dense width %d is too large", who, N);
    if (!c || !b || !coarse_row_offsets || ((!a || !coarse_row_blocks) && coarse_nnz > 0))
        return fail(BSA_ERR_INVALID, "%s: null pointer argument", who);
    int rc = check_schedule(sched, sched_wgs, sched_waves, batches, who);
    if (rc) return rc;
    if (sched_waves > 4)
        return fail(BSA_ERR_INVALID, "%s: at most 4 waves per workgroup (64 x 64 fp32 tiles meet in LDS), got %d", who,
                    sched_waves);
    bsa::Block64Args p{a, b, c, coarse_row_blocks, coarse_row_offsets, sched, coarse_rows, coarse_cols, coarse_nnz,
                       sched_wgs, sched_waves, batches, N, sparse_batches != batches};
    return check_launch(bsa::launch_dsd_block64(dtype, p, (hipStream_t)stream), who);
}

int64_t bsa_run_schedule_bytes(int mask_rows, int nnz)
{
    if (mask_rows < 1 || nnz < 0) return 0;
    return (int64_t)mask_rows * bsa::RUN_RECORD_BYTES + (((int64_t)nnz + 3) & ~(int64_t)3);
}

int bsa_run_schedule_build(const int32_t *row_blocks, const int32_t *row_offsets, int mask_rows, int nnz,
                           int target_pairs, int max_strips, void *sched, int64_t sched_bytes,
                           int32_t *counts_out, void *stream)
{
    const char *who = "bsa_run_schedule_build";
    if (mask_rows < 1 || mask_rows > 32767) return fail(BSA_ERR_INVALID, "%s: %d block rows outside [1, 32767]", who, mask_rows);
    if (nnz < 0) return fail(BSA_ERR_INVALID, "%s: nnz %d < 0", who, nnz);
    if (target_pairs < 1) return fail(BSA_ERR_INVALID, "%s: target_pairs %d < 1", who, target_pairs);
    if (max_strips < 1 || max_strips > bsa::RUN_MAX_STRIPS)
        return fail(BSA_ERR_INVALID, "%s: max_strips %d outside [1, %d]", who, max_strips, bsa::RUN_MAX_STRIPS);
    if (!row_offsets || !sched || !counts_out || (!row_blocks && nnz > 0))
        return fail(BSA_ERR_INVALID, "%s: null pointer argument", who);
    if (sched_bytes < bsa_run_schedule_bytes(mask_rows, nnz))
        return fail(BSA_ERR_INVALID, "%s: the schedule needs %lld bytes, got %lld", who,
                    (long long)bsa_run_schedule_bytes(mask_rows, nnz), (long long)sched_bytes);
    if (target_pairs > (nnz > 0 ? nnz : 1)) target_pairs = nnz > 0 ? nnz : 1;    // one run at most: no sum in the build overflows
    return check_launch(bsa::launch_run_schedule_build(row_blocks, row_offsets, mask_rows, nnz, target_pairs, max_strips,
                                                       sched, counts_out, (hipStream_t)stream), who);
}

int bsa_matmul_dsd_runs(int dtype, const void *a, const void *b, void *c,
                        const int32_t *row_blocks, const int32_t *row_offsets,
                        const void *run_sched, int n_runs, int run_strips, int run_pairs, int waves,
                        int mask_rows, int mask_cols, int nnz, int batches, int sparse_batches,
                        int N, void *stream)
{
    const char *who = "bsa_matmul_dsd_runs";
    if (dtype != BSA_F16 && dtype != BSA_BF16)
        return fail(BSA_ERR_UNSUPPORTED, "%s: fp16 (dtype 1) and bf16 (dtype 2) are built, got %d", who, dtype);
    if (mask_rows < 1 || mask_rows > 32767 || mask_cols < 1 || mask_cols > 65535)
        return fail(BSA_ERR_INVALID, "%s: mask shape %d x %d out of range", who, mask_rows, mask_cols);
    if (nnz < 0 || (long long)nnz > (long long)mask_rows * mask_cols)
        return fail(BSA_ERR_INVALID, "%s: nnz %d does not fit a %d x %d mask", who, nnz, mask_rows, mask_cols);
    if (batches < 1 || (sparse_batches != batches && sparse_batches != 1))
        return fail(BSA_ERR_INVALID, "%s: batches %d, sparse_batches %d", who, batches, sparse_batches);
    if (N < 64 || N % 64)
        return fail(BSA_ERR_UNSUPPORTED, "%s: the dense width must be a positive multiple of 64, got %d (use bsa_matmul)", who, N);
    if (N / 64 > 65535) return fail(BSA_ERR_INVALID, "%s: dense width %d is too large", who, N);
    if (!c || !b || !row_offsets || !run_sched || ((!a || !row_blocks) && nnz > 0))
        return fail(BSA_ERR_INVALID, "%s: null pointer argument", who);
    if (n_runs < 1 || n_runs > mask_rows)
        return fail(BSA_ERR_INVALID, "%s: %d runs for %d block rows (a table that bsa_run_schedule_build reports as not "
                    "eligible has none: use bsa_matmul)", who, n_runs, mask_rows);
    if (waves < 1 || waves > bsa::RUN_MAX_WAVES)
        return fail(BSA_ERR_INVALID, "%s: %d waves per workgroup outside [1, %d]", who, waves, bsa::RUN_MAX_WAVES);
    if (run_strips < 0 || run_strips > bsa::RUN_MAX_STRIPS || run_strips > 4 * waves)
        return fail(BSA_ERR_INVALID, "%s: %d strips per run: at most %d, and 4 per wave", who, run_strips, bsa::RUN_MAX_STRIPS);
    if (run_pairs < 0 || run_pairs > 64 * waves)
        return fail(BSA_ERR_INVALID, "%s: a run of %d pairs needs more than %d waves (64 pairs each)", who, run_pairs, waves);
    if ((long long)n_runs * ((batches + 7) / 8) > (1LL << 27))
        return fail(BSA_ERR_INVALID, "%s: %d runs x %d batch entries do not fit one launch", who, n_runs, batches);
    bsa::RunsArgs p{a, b, c, row_blocks, row_offsets, run_sched, n_runs, waves, run_strips < 1 ? 1 : run_strips,
                    mask_rows, mask_cols, nnz, batches, N, sparse_batches != batches};
    return check_launch(bsa::launch_dsd_runs(dtype, p, (hipStream_t)stream), who);
}

static int check_softmax(const char *who, int dtype, const void *p0, const void *p1, const void *p2,
                         const int32_t *blocks, const int32_t *offsets, const int32_t *sched,
                         int sched_wgs, int sched_waves, int mask_rows, int mask_cols, int nnz, int batches)
{
    if (dtype != BSA_F32 && dtype != BSA_F16 && dtype != BSA_BF16)
        return fail(BSA_ERR_UNSUPPORTED, "%s: unsupported dtype %d (fp32 = 0, fp16 = 1, bf16 = 2)", who, dtype);
    if (!p0 || !p1 || !p2 || !blocks || !offsets) return fail(BSA_ERR_INVALID, "%s: null pointer argument", who);
    if (mask_rows < 1 || mask_rows > 32767 || mask_cols < 1 || mask_cols > 65535)
        return fail(BSA_ERR_INVALID, "%s: mask shape %d x %d out of range", who, mask_rows, mask_cols);
    if (nnz < 0 || (long long)nnz > (long long)mask_rows * mask_cols)
        return fail(BSA_ERR_INVALID, "%s: nnz %d does not fit a %d x %d mask", who, nnz, mask_rows, mask_cols);
    if (batches < 1) return fail(BSA_ERR_INVALID, "%s: batches %d < 1", who, batches);
    return check_schedule(sched, sched_wgs, sched_waves, batches, who);
}

int bsa_softmax_forward(int dtype, const void *x, void *y,
                        const int32_t *row_blocks, const int32_t *row_offsets,
                        const int32_t *sched, int sched_wgs, int sched_waves,
                        int mask_rows, int mask_cols, int nnz, int batches,
                        float scale, int causal, void *stream)
{
    int rc = check_softmax("bsa_softmax_forward", dtype, x, y, y, row_blocks, row_offsets, sched, sched_wgs,
                           sched_waves, mask_rows, mask_cols, nnz, batches);
    if (rc) return rc;
    if (nnz == 0) return BSA_OK;
    bsa::SoftmaxArgs p{x, nullptr, y, row_blocks, sched, mask_rows, sched_wgs, sched_waves, nnz, batches, scale, causal != 0};
    return check_launch(bsa::launch_softmax_forward(dtype, p, (hipStream_t)stream), "bsa_softmax_forward");
}

int bsa_softmax_backward(int dtype, const void *y, const void *dy, void *dx,
                         const int32_t *row_blocks, const int32_t *row_offsets,
                         const int32_t *sched, int sched_wgs, int sched_waves,
                         int mask_rows, int mask_cols, int nnz, int batches,
                         float scale, void *stream)
{
    int rc = check_softmax("bsa_softmax_backward", dtype, y, dy, dx, row_blocks, row_offsets, sched, sched_wgs,
                           sched_waves, mask_rows, mask_cols, nnz, batches);
    if (rc) return rc;
    if (nnz == 0) return BSA_OK;
    bsa::SoftmaxArgs p{y, dy, dx, row_blocks, sched, mask_rows, sched_wgs, sched_waves, nnz, batches, scale, false};
    return check_launch(bsa::launch_softmax_backward(dtype, p, (hipStream_t)stream), "bsa_softmax_backward");
}

static int check_attention(const char *who, int dtype, int head_dim, const int32_t *row_blocks,
                           const int32_t *row_offsets, const int32_t *sched, int sched_wgs, int sched_waves,
                           int mask_rows, int mask_cols, int nnz, int batches)
{
    if (dtype != BSA_F16 && dtype != BSA_BF16)
        return fail(BSA_ERR_UNSUPPORTED, "%s: only fp16 (dtype 1) and bf16 (dtype 2) are built, got %d", who, dtype);
    if (head_dim != 64 && head_dim != 128)
        return fail(BSA_ERR_UNSUPPORTED, "%s: head_dim 64 and 128 are built, got %d", who, head_dim);
    if (!row_offsets || (!row_blocks && nnz > 0)) return fail(BSA_ERR_INVALID, "%s: null pointer argument", who);
    if (mask_rows < 1 || mask_rows > 32767 || mask_cols < 1 || mask_cols > 65535)
        return fail(BSA_ERR_INVALID, "%s: mask shape %d x %d out of range", who, mask_rows, mask_cols);
    if (nnz < 0 || (long long)nnz > (long long)mask_rows * mask_cols)
        return fail(BSA_ERR_INVALID, "%s: nnz %d does not fit a %d x %d mask", who, nnz, mask_rows, mask_cols);
    if (batches < 1) return fail(BSA_ERR_INVALID, "%s: batches %d < 1", who, batches);
    return check_schedule(sched, sched_wgs, sched_waves, batches, who);
}

static void fill_attention(bsa::AttentionArgs &p, int dtype, const void *q, const void *k, const void *v,
                           const int32_t *blocks, const int32_t *sched, int groups, int sched_wgs, int sched_waves,
                           int mask_rows, int mask_cols, int nnz, int batches, int head_dim, float scale, int causal)
{
    p.q = q;
    p.k = k;
    p.v = v;
    p.blocks = blocks;
    p.sched = sched;
    p.groups = groups;
    p.sched_wgs = sched_wgs;
    p.sched_waves = sched_waves;
    p.mask_rows = mask_rows;
    p.mask_cols = mask_cols;
    p.nnz = nnz;
    p.batches = batches;
    p.head_dim = head_dim;
    p.scale = scale;
    p.causal = causal != 0;
    p.bf16 = dtype == BSA_BF16;
}

size_t bsa_attention_workspace_bytes(int sched_tile_slots, int sched_split_groups, int batches, int head_dim)
{
    if (batches < 1 || (head_dim != 64 && head_dim != 128)) return 0;
    return bsa::attention_workspace_bytes(sched_tile_slots, sched_split_groups, batches, head_dim);
}

int bsa_attention_forward(int dtype, const void *q, const void *k, const void *v, void *out, float *lse,
                          const int32_t *row_blocks, const int32_t *row_offsets,
                          const int32_t *sched, int sched_wgs, int sched_waves,
                          int sched_tile_slots, int sched_split_groups, void *workspace, size_t workspace_bytes,
                          int mask_rows, int mask_cols, int nnz, int batches, int head_dim,
                          float scale, int causal, void *stream)
{
    const char *who = "bsa_attention_forward";
    int rc = check_attention(who, dtype, head_dim, row_blocks, row_offsets, sched, sched_wgs, sched_waves,
                             mask_rows, mask_cols, nnz, batches);
    if (rc) return rc;
    if (!q || !k || !v || !out) return fail(BSA_ERR_INVALID, "%s: null pointer argument", who);
    if (sched_tile_slots < 0 || sched_split_groups < 0 || (sched_tile_slots > 0) != (sched_split_groups > 0))
        return fail(BSA_ERR_INVALID, "%s: schedule split counts %d, %d are inconsistent", who, sched_tile_slots,
                    sched_split_groups);
    const size_t ws_need = bsa_attention_workspace_bytes(sched_tile_slots, sched_split_groups, batches, head_dim);
    if (ws_need > 0 && (!workspace || workspace_bytes < ws_need))
        return fail(BSA_ERR_INVALID, "%s: workspace of %zu bytes needed, %zu given", who, ws_need, workspace_bytes);
    bsa::AttentionArgs p;
    fill_attention(p, dtype, q, k, v, row_blocks, sched, mask_rows, sched_wgs, sched_waves, mask_rows, mask_cols, nnz,
                   batches, head_dim, scale, causal);
    p.out = out;
    p.lse = lse;
    p.tile_slots = sched_tile_slots;
    p.split_groups = sched_split_groups;
    p.workspace = workspace;
    return check_launch(bsa::launch_attention_forward(p, (hipStream_t)stream), who);
}

static int check_split_workspace(const char *who, int tile_slots, int split_groups)
{
    if (tile_slots < 0 || split_groups < 0 || (tile_slots > 0) != (split_groups > 0))
        return fail(BSA_ERR_INVALID, "%s: schedule split counts %d, %d are inconsistent", who, tile_slots, split_groups);
    return BSA_OK;
}

size_t bsa_attention_backward_workspace_bytes(int row_tile_slots, int row_split_groups, int col_tile_slots,
                                              int col_split_groups, int batches, int head_dim)
{
    if (batches < 1 || (head_dim != 64 && head_dim != 128)) return 0;
    return bsa::attention_backward_workspace_bytes(row_tile_slots, row_split_groups, col_tile_slots, col_split_groups,
                                                   batches, head_dim);
}

int bsa_attention_backward_scores(int dtype, const void *q, const void *k, const void *v, const void *dout,
                                  const void *out, const float *lse, void *p_out, void *ds_out, void *dq_out,
                                  const int32_t *row_blocks, const int32_t *row_offsets,
                                  const int32_t *sched, int sched_wgs, int sched_waves,
                                  int sched_tile_slots, int sched_split_groups, void *workspace, size_t workspace_bytes,
                                  int mask_rows, int mask_cols, int nnz, int batches, int head_dim,
                                  float scale, int causal, void *stream)
{
    const char *who = "bsa_attention_backward_scores";
    int rc = check_attention(who, dtype, head_dim, row_blocks, row_offsets, sched, sched_wgs, sched_waves,
                             mask_rows, mask_cols, nnz, batches);
    if (rc) return rc;
    if (nnz == 0 && !dq_out) return BSA_OK;      // no blocks to write
    if (!q || !k || !v || !dout || !out || !lse) return fail(BSA_ERR_INVALID, "%s: null pointer argument", who);
    if ((p_out == nullptr) != (ds_out == nullptr))
        return fail(BSA_ERR_INVALID, "%s: p_out and ds_out go together", who);
    if (!p_out && !dq_out) return fail(BSA_ERR_INVALID, "%s: no output asked for", who);
    rc = check_split_workspace(who, sched_tile_slots, sched_split_groups);
    if (rc) return rc;
    const size_t ws_need = dq_out ? bsa_attention_backward_workspace_bytes(sched_tile_slots, sched_split_groups, 0, 0,
                                                                           batches, head_dim) : 0;
    if (ws_need > 0 && (!workspace || workspace_bytes < ws_need))
        return fail(BSA_ERR_INVALID, "%s: workspace of %zu bytes needed, %zu given", who, ws_need, workspace_bytes);
    bsa::AttentionArgs p;
    fill_attention(p, dtype, q, k, v, row_blocks, sched, mask_rows, sched_wgs, sched_waves, mask_rows, mask_cols, nnz,
                   batches, head_dim, scale, causal);
    p.out = const_cast<void *>(out);
    p.lse = const_cast<float *>(lse);
    p.dout = dout;
    p.p_out = p_out;
    p.ds_out = ds_out;
    p.dq_out = dq_out;
    p.tile_slots = sched_tile_slots;
    p.split_groups = sched_split_groups;
    p.workspace = workspace;
    return check_launch(bsa::launch_attention_backward_scores(p, (hipStream_t)stream), who);
}

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
                           float scale, int causal, void *stream)
{
    const char *who = "bsa_attention_backward";
    int rc = check_attention(who, dtype, head_dim, row_blocks, row_offsets, row_sched, row_sched_wgs, row_sched_waves,
                             mask_rows, mask_cols, nnz, batches);
    if (rc) return rc;
    if (head_dim != 64) return fail(BSA_ERR_UNSUPPORTED, "%s: head_dim 64 is built, got %d", who, head_dim);
    if (!col_offsets || (!col_blocks && nnz > 0)) return fail(BSA_ERR_INVALID, "%s: null pointer argument", who);
    rc = check_schedule(col_sched, col_sched_wgs, col_sched_waves, batches, who);
    if (rc) return rc;
    if (!q || !k || !v || !dout || !out || !lse || !dq_out || !dk_out || !dv_out || !delta_ws)
        return fail(BSA_ERR_INVALID, "%s: null pointer argument", who);
    rc = check_split_workspace(who, row_tile_slots, row_split_groups);
    if (rc) return rc;
    rc = check_split_workspace(who, col_tile_slots, col_split_groups);
    if (rc) return rc;
    const size_t row_bytes = bsa_attention_backward_workspace_bytes(row_tile_slots, row_split_groups, 0, 0, batches, head_dim);
    const size_t ws_need = bsa_attention_backward_workspace_bytes(row_tile_slots, row_split_groups, col_tile_slots,
                                                                  col_split_groups, batches, head_dim);
    if (ws_need > 0 && (!workspace || workspace_bytes < ws_need))
        return fail(BSA_ERR_INVALID, "%s: workspace of %zu bytes needed, %zu given", who, ws_need, workspace_bytes);
    bsa::AttentionArgs p;
    fill_attention(p, dtype, q, k, v, row_blocks, row_sched, mask_rows, row_sched_wgs, row_sched_waves, mask_rows,
                   mask_cols, nnz, batches, head_dim, scale, causal);
    p.out = const_cast<void *>(out);
    p.lse = const_cast<float *>(lse);
    p.dout = dout;
    p.dq_out = dq_out;
    p.delta = delta_ws;
    p.tile_slots = row_tile_slots;
    p.split_groups = row_split_groups;
    p.workspace = workspace;
    rc = check_launch(bsa::launch_attention_backward_scores(p, (hipStream_t)stream), who);
    if (rc) return rc;
    p.blocks = col_blocks;
    p.sched = col_sched;
    p.groups = mask_cols;
    p.sched_wgs = col_sched_wgs;
    p.sched_waves = col_sched_waves;
    p.tile_slots = col_tile_slots;
    p.split_groups = col_split_groups;
    p.workspace = workspace ? (char *)workspace + row_bytes : nullptr;
    p.dk_out = dk_out;
    p.dv_out = dv_out;
    return check_launch(bsa::launch_attention_backward_dkdv(p, (hipStream_t)stream), who);
}

}  // extern "C"
