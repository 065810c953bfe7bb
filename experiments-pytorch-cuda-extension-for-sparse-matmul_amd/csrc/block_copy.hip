// Dense matrix <-> stack of its stored 32x32 blocks, for gfx950.
//
// Replaces SparseLayout.to_sparse / to_dense (sparse/layout.py:40-57), which the reference writes
// as Python loops over the blocks of a CPU-side index list.  One wavefront moves one block per
// batch entry: the dense side is 32 rows of 32 elements (64 or 128 contiguous bytes each), the
// sparse side one contiguous 2 or 4 KB piece; every lane moves 16-byte pieces, and both sides are
// touched once (non-temporal).  to_dense walks every CELL of the mask and writes zeros where no
// block is stored, so the result needs no separate fill.
#include "bsa_device.hpp"
#include "bsa_internal.hpp"

namespace bsa {

constexpr int BC_WAVES = 4;

// piece p (16 bytes) of a block: row p / (2 ES), 16-byte column piece p % (2 ES)
template <int ES>
__device__ __forceinline__ size_t dense_piece_offset(int p, size_t row_bytes)
{
    return (size_t)(p / (2 * ES)) * row_bytes + 16u * (unsigned)(p % (2 * ES));
}

template <int ES>
__global__ __launch_bounds__(64 * BC_WAVES) void to_sparse_kernel(
    const unsigned char *__restrict__ dense, unsigned char *__restrict__ sparse,
    const BlockDesc *__restrict__ blocks, int nnz, int batches, int R, int C)
{
    const int idx = (int)blockIdx.x * BC_WAVES + wave_id();
    if (idx >= nnz) return;
    const int l = lane_id();
    const BlockDesc d = blocks[idx];
    const size_t row_bytes = (size_t)C * BS * ES;
    for (int b = (int)blockIdx.y; b < batches; b += (int)gridDim.y) {
        const unsigned char *src = dense + ((size_t)b * R * BS + (size_t)BS * d.row()) * row_bytes + (size_t)BS * ES * d.col();
        unsigned char *dst = sparse + ((size_t)b * nnz + d.idx) * BS2 * ES;
#pragma unroll
        for (int q = 0; q < ES; ++q) {
            const int p = l + WAVE * q;
            stg16_stream(dst + 16 * p, ldg16_stream(src + dense_piece_offset<ES>(p, row_bytes)));
        }
    }
}

// ordinal_of[cell] = number of stored blocks in front of the cell in row-major order (what
// layout_build_kernel leaves in its workspace): the block index of a stored cell
template <int ES>
__global__ __launch_bounds__(64 * BC_WAVES) void to_dense_kernel(
    const unsigned char *__restrict__ sparse, unsigned char *__restrict__ dense,
    const uint8_t *__restrict__ mask, const int *__restrict__ ordinal_of, int nnz, int batches, int R, int C)
{
    const int cell = (int)blockIdx.x * BC_WAVES + wave_id();
    if (cell >= R * C) return;
    const int l = lane_id();
    const int r = cell / C, c = cell - r * C;
    const bool stored = mask[cell] != 0;
    const int idx = stored ? ordinal_of[cell] : 0;
    const size_t row_bytes = (size_t)C * BS * ES;
    for (int b = (int)blockIdx.y; b < batches; b += (int)gridDim.y) {
        unsigned char *dst = dense + ((size_t)b * R * BS + (size_t)BS * r) * row_bytes + (size_t)BS * ES * c;
        const unsigned char *src = sparse + ((size_t)b * nnz + idx) * BS2 * ES;
#pragma unroll
        for (int q = 0; q < ES; ++q) {
            const int p = l + WAVE * q;
            const uint4 v = stored ? ldg16_stream(src + 16 * p) : make_uint4(0, 0, 0, 0);
            stg16_stream(dst + dense_piece_offset<ES>(p, row_bytes), v);
        }
    }
}

hipError_t launch_to_sparse(int elem_size, const void *dense, void *sparse, const int32_t *row_blocks,
                            int nnz, int batches, int R, int C, hipStream_t st)
{
    dim3 grid((unsigned)((nnz + BC_WAVES - 1) / BC_WAVES), (unsigned)(batches < 65535 ? batches : 65535)), block(64 * BC_WAVES);
    if (elem_size == 2)
        to_sparse_kernel<2><<<grid, block, 0, st>>>((const unsigned char *)dense, (unsigned char *)sparse,
                                                   (const BlockDesc *)row_blocks, nnz, batches, R, C);
    else
        to_sparse_kernel<4><<<grid, block, 0, st>>>((const unsigned char *)dense, (unsigned char *)sparse,
                                                   (const BlockDesc *)row_blocks, nnz, batches, R, C);
    return hipGetLastError();
}

hipError_t launch_to_dense(int elem_size, const void *sparse, void *dense, const uint8_t *mask,
                           const int32_t *ordinal_of, int nnz, int batches, int R, int C, hipStream_t st)
{
    dim3 grid((unsigned)((R * C + BC_WAVES - 1) / BC_WAVES), (unsigned)(batches < 65535 ? batches : 65535)), block(64 * BC_WAVES);
    if (elem_size == 2)
        to_dense_kernel<2><<<grid, block, 0, st>>>((const unsigned char *)sparse, (unsigned char *)dense, mask,
                                                  ordinal_of, nnz, batches, R, C);
    else
        to_dense_kernel<4><<<grid, block, 0, st>>>((const unsigned char *)sparse, (unsigned char *)dense, mask,
                                                  ordinal_of, nnz, batches, R, C);
    return hipGetLastError();
}

}  // namespace bsa
