/*
 * Plain-C block-walk restatement of the block-sparse kernels (CPU oracle).
 *
 * TEST INFRASTRUCTURE ONLY: the shipped library never links or loads this file.
 *
 * Where the dense numpy oracle states WHAT the operators mean, this file
 * restates HOW the reference kernels get there: walk the block table of a
 * group, gather one 32x32 sparse block and one 32-wide dense tile per entry,
 * multiply-accumulate.  The two must agree; the tests check that.
 *
 *   table format        sparse/layout.py:21-36, sparse/native/sparse_layout.cuh:13-21
 *   SDD  walk           sparse/native/sparse_smm_gpu.cu:33-94   (one block per work item)
 *   DSD  walk           sparse/native/sparse_smm_gpu.cu:118-180 (group = output block row)
 *   DDS  walk           sparse/native/sparse_smm_gpu.cu:204-266 (group = output block column)
 *   softmax fwd / bwd   sparse_softmax.cu:130-153 / :190-203
 *
 * Differences from the reference, all deliberate: the contraction index of a
 * transposed sparse operand is the block ROW for column groups and the block
 * COLUMN for row groups (the reference always uses one of them, lines 134 and
 * 219); the column is decoded from 16 bits; accumulation is in double; the
 * softmax has a scale and an optional causal mask; an empty group yields zeros.
 *
 * Inputs are float (fp16 data is widened exactly by the caller), outputs double.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#define BS 32
#define BS2 (BS * BS)

static inline int blk_idx(const int32_t *blocks, int p) { return blocks[2 * p]; }
static inline int blk_row(const int32_t *blocks, int p) { return (int)((uint32_t)blocks[2 * p + 1] >> 16); }
static inline int blk_col(const int32_t *blocks, int p) { return blocks[2 * p + 1] & 0xFFFF; }

/* Tables from a 0/1 byte mask.  Returns nnz.  blocks needs 2*R*C ints at most. */
int bsa_oracle_layout(const uint8_t *mask, int R, int C, int transpose,
                      int32_t *blocks, int32_t *offsets)
{
    int n = 0;
    int G = transpose ? C : R, L = transpose ? R : C;
    offsets[0] = 0;
    for (int g = 0; g < G; ++g) {
        for (int l = 0; l < L; ++l) {
            int r = transpose ? l : g, c = transpose ? g : l;
            if (!mask[(size_t)r * C + c]) continue;
            int ordinal = 0; /* row-major ordinal among the nonzeros */
            for (size_t q = 0; q < (size_t)r * C + c; ++q) ordinal += mask[q] != 0;
            blocks[2 * n] = ordinal;
            blocks[2 * n + 1] = (int32_t)(((uint32_t)r << 16) + (uint32_t)c);
            ++n;
        }
        offsets[g + 1] = n;
    }
    return n;
}

/* element (i, k) of op(X) for a dense X stored [rows, cols] (ld = cols) */
static inline double dense_at(const float *x, int ld, int tr, int i, int k)
{
    return tr ? (double)x[(size_t)k * ld + i] : (double)x[(size_t)i * ld + k];
}

/* c[b, idx] = op(a)[32r:32r+32, :] * op(b)[:, 32c:32c+32] for every table entry */
void bsa_oracle_sdd(const float *a, const float *b, double *c, const int32_t *blocks,
                    int nnz, int batches, int M, int N, int K, int tr_a, int tr_b)
{
    int lda = tr_a ? M : K, ldb = tr_b ? K : N;
    for (int bt = 0; bt < batches; ++bt) {
        const float *ab = a + (size_t)bt * M * K, *bb = b + (size_t)bt * N * K;
        double *cb = c + (size_t)bt * nnz * BS2;
        for (int p = 0; p < nnz; ++p) {
            int r = blk_row(blocks, p), cc = blk_col(blocks, p);
            double *out = cb + (size_t)blk_idx(blocks, p) * BS2;
            for (int i = 0; i < BS; ++i)
                for (int j = 0; j < BS; ++j) {
                    double acc = 0.0;
                    for (int k = 0; k < K; ++k)
                        acc += dense_at(ab, lda, tr_a, r * BS + i, k) *
                               dense_at(bb, ldb, !tr_b, cc * BS + j, k);
                    out[i * BS + j] = acc;
                }
        }
    }
}

/* c[b, 32g:32g+32, :] = sum over group g of op(S_blk) * op(b)[32*kblk:+32, :]
 * groups are rows of S when !tr_a (kblk = block col) and columns when tr_a (kblk = block row) */
void bsa_oracle_dsd(const float *s, const float *b, double *c, const int32_t *blocks,
                    const int32_t *offsets, int groups, int nnz, int batches,
                    int N, int K, int tr_a, int tr_b)
{
    int M = groups * BS, ldb = tr_b ? K : N;
    for (int bt = 0; bt < batches; ++bt) {
        const float *sb = s + (size_t)bt * nnz * BS2, *bb = b + (size_t)bt * N * K;
        double *cb = c + (size_t)bt * M * N;
        memset(cb, 0, sizeof(double) * (size_t)M * N);
        for (int g = 0; g < groups; ++g)
            for (int p = offsets[g]; p < offsets[g + 1]; ++p) {
                const float *blk = sb + (size_t)blk_idx(blocks, p) * BS2;
                int kb = tr_a ? blk_row(blocks, p) : blk_col(blocks, p);
                for (int i = 0; i < BS; ++i)
                    for (int k = 0; k < BS; ++k) {
                        double sv = tr_a ? (double)blk[k * BS + i] : (double)blk[i * BS + k];
                        for (int n = 0; n < N; ++n)
                            cb[(size_t)(g * BS + i) * N + n] +=
                                sv * dense_at(bb, ldb, tr_b, kb * BS + k, n);
                    }
            }
    }
}

/* c[b, :, 32g:32g+32] = sum over group g of op(a)[:, 32*kblk:+32] * op(S_blk)
 * groups are columns of S when !tr_b (kblk = block row) and rows when tr_b (kblk = block col) */
void bsa_oracle_dds(const float *a, const float *s, double *c, const int32_t *blocks,
                    const int32_t *offsets, int groups, int nnz, int batches,
                    int M, int K, int tr_a, int tr_b)
{
    int N = groups * BS, lda = tr_a ? M : K;
    for (int bt = 0; bt < batches; ++bt) {
        const float *ab = a + (size_t)bt * M * K, *sb = s + (size_t)bt * nnz * BS2;
        double *cb = c + (size_t)bt * M * N;
        memset(cb, 0, sizeof(double) * (size_t)M * N);
        for (int g = 0; g < groups; ++g)
            for (int p = offsets[g]; p < offsets[g + 1]; ++p) {
                const float *blk = sb + (size_t)blk_idx(blocks, p) * BS2;
                int kb = tr_b ? blk_col(blocks, p) : blk_row(blocks, p);
                for (int m = 0; m < M; ++m)
                    for (int k = 0; k < BS; ++k) {
                        double av = dense_at(ab, lda, tr_a, m, kb * BS + k);
                        for (int j = 0; j < BS; ++j) {
                            double sv = tr_b ? (double)blk[j * BS + k] : (double)blk[k * BS + j];
                            cb[(size_t)m * N + g * BS + j] += av * sv;
                        }
                    }
            }
    }
}

/* y = softmax(scale * x [+ causal mask]) over the stored blocks of every row */
void bsa_oracle_softmax_fwd(const float *x, double *y, const int32_t *blocks,
                            const int32_t *offsets, int groups, int nnz, int batches,
                            double scale, int causal)
{
    for (int bt = 0; bt < batches; ++bt) {
        const float *xb = x + (size_t)bt * nnz * BS2;
        double *yb = y + (size_t)bt * nnz * BS2;
        for (int g = 0; g < groups; ++g)
            for (int r = 0; r < BS; ++r) {
                int grow = g * BS + r;
                double mx = -INFINITY, sum = 0.0;
                for (int p = offsets[g]; p < offsets[g + 1]; ++p) {
                    const float *row = xb + (size_t)blk_idx(blocks, p) * BS2 + r * BS;
                    for (int j = 0; j < BS; ++j) {
                        if (causal && blk_col(blocks, p) * BS + j > grow) continue;
                        double v = scale * (double)row[j];
                        if (v > mx) mx = v;
                    }
                }
                for (int p = offsets[g]; p < offsets[g + 1]; ++p) {
                    const float *row = xb + (size_t)blk_idx(blocks, p) * BS2 + r * BS;
                    double *out = yb + (size_t)blk_idx(blocks, p) * BS2 + r * BS;
                    for (int j = 0; j < BS; ++j) {
                        int masked = causal && blk_col(blocks, p) * BS + j > grow;
                        out[j] = (masked || mx == -INFINITY) ? 0.0 : exp(scale * (double)row[j] - mx);
                        sum += out[j];
                    }
                }
                for (int p = offsets[g]; p < offsets[g + 1]; ++p) {
                    double *out = yb + (size_t)blk_idx(blocks, p) * BS2 + r * BS;
                    for (int j = 0; j < BS; ++j) out[j] = sum > 0.0 ? out[j] / sum : 0.0;
                }
            }
    }
}

/* dx = scale * (dy - sum(dy * y)) * y over the stored blocks of every row */
void bsa_oracle_softmax_bwd(const float *y, const float *dy, double *dx, const int32_t *blocks,
                            const int32_t *offsets, int groups, int nnz, int batches,
                            double scale)
{
    for (int bt = 0; bt < batches; ++bt) {
        const float *yb = y + (size_t)bt * nnz * BS2, *dyb = dy + (size_t)bt * nnz * BS2;
        double *dxb = dx + (size_t)bt * nnz * BS2;
        for (int g = 0; g < groups; ++g)
            for (int r = 0; r < BS; ++r) {
                double dot = 0.0;
                for (int p = offsets[g]; p < offsets[g + 1]; ++p) {
                    size_t o = (size_t)blk_idx(blocks, p) * BS2 + r * BS;
                    for (int j = 0; j < BS; ++j) dot += (double)dyb[o + j] * (double)yb[o + j];
                }
                for (int p = offsets[g]; p < offsets[g + 1]; ++p) {
                    size_t o = (size_t)blk_idx(blocks, p) * BS2 + r * BS;
                    for (int j = 0; j < BS; ++j)
                        dxb[o + j] = scale * ((double)dyb[o + j] - dot) * (double)yb[o + j];
                }
            }
    }
}
