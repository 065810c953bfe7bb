"""Block-index tables and dense<->block-stack converters (CPU oracle).

TEST INFRASTRUCTURE ONLY: nothing shipped imports this file.

Two independent builders of the same tables are kept here on purpose:

* :func:`create_layout` restates the vectorised construction of the reference,
  ``sparse/layout.py:14-38`` (nonzero -> cumsum ordinal -> packed position ->
  offset table by counting), in numpy.
* :func:`create_layout_bruteforce` derives the same tables from their meaning
  with plain double loops (no cumsum, no nonzero).

The tests require both to agree bit for bit with each other, with the device
builder and with hand-derived known answers.

Table format (the bit-exact contract, ``sparse/layout.py:21-36`` and the device
view ``sparse/native/sparse_layout.cuh:13-21``):

``blocks``        int32[2*nnz], interleaved pairs ``(idx, packed_pos)`` where
                  ``idx`` is the row-major ordinal of the block among the
                  nonzero blocks and ``packed_pos = (row << 16) + col``.
``offset_table``  int32[G+1], first entry of every group (CSR row pointer for
                  the row layout, CSC column pointer for the column layout).

The pattern is taken as a 0/1 integer mask; a bool mask is defined to give the
tables of the equivalent 0/1 integer mask (the reference's own arithmetic
saturates on bool input, which is a defect, not a contract).
"""
import numpy as np

BLOCK = 32


def _as_mask(pattern) -> np.ndarray:
    mask = np.asarray(pattern)
    if mask.ndim != 2:
        raise ValueError("pattern must be 2-D")
    return (mask != 0).astype(np.int64)


def create_layout(pattern, transpose: bool = False):
    """numpy restatement of ``SparseLayout._create_layout`` (sparse/layout.py:14-38)."""
    mask = _as_mask(pattern)
    n_cols = mask.shape[1]
    if transpose:
        # nonzero of the transposed mask: column-major order (layout.py:16-17)
        cols, rows = np.nonzero(mask.T)
    else:
        rows, cols = np.nonzero(mask)                      # layout.py:19
    ordinal = np.cumsum(mask.reshape(-1))                  # layout.py:22
    idx = ordinal[rows * n_cols + cols] - 1                # layout.py:23
    packed_pos = (rows << 16) + cols                       # layout.py:25
    blocks = np.stack((idx, packed_pos), axis=1).astype(np.int32).reshape(-1)  # :26

    keys = (cols if transpose else rows) + 1               # layout.py:30
    table_size = mask.shape[1 if transpose else 0] + 1     # layout.py:33
    counts = np.zeros(table_size, dtype=np.int64)
    np.add.at(counts, keys, 1)                             # layout.py:34-35
    offset_table = np.cumsum(counts).astype(np.int32)      # layout.py:36
    return blocks, offset_table


def create_layout_bruteforce(pattern, transpose: bool = False):
    """Same tables from their definition, with explicit loops."""
    mask = _as_mask(pattern)
    n_rows, n_cols = mask.shape
    ordinal = {}
    for r in range(n_rows):
        for c in range(n_cols):
            if mask[r, c]:
                ordinal[(r, c)] = len(ordinal)
    blocks, offsets = [], [0]
    if transpose:
        for c in range(n_cols):
            for r in range(n_rows):
                if mask[r, c]:
                    blocks += [ordinal[(r, c)], r * 65536 + c]
            offsets.append(len(blocks) // 2)
    else:
        for r in range(n_rows):
            for c in range(n_cols):
                if mask[r, c]:
                    blocks += [ordinal[(r, c)], r * 65536 + c]
            offsets.append(len(blocks) // 2)
    return (np.asarray(blocks, dtype=np.int32).reshape(-1),
            np.asarray(offsets, dtype=np.int32))


def sparse_positions(pattern) -> np.ndarray:
    """``torch.nonzero(pattern)`` of sparse/layout.py:8 : int64 [nnz, 2], row-major."""
    mask = _as_mask(pattern)
    rows, cols = np.nonzero(mask)
    return np.stack((rows, cols), axis=1).astype(np.int64)


def decode_blocks(blocks: np.ndarray):
    """Device-side decode, sparse/native/sparse_layout.cuh:15-17, with the column
    taken from the full low 16 bits (the reference masks 8 bits only, which
    wraps beyond 256 block columns)."""
    pairs = np.asarray(blocks).reshape(-1, 2)
    return pairs[:, 0], pairs[:, 1] >> 16, pairs[:, 1] & 0xFFFF


def to_sparse(pattern, x: np.ndarray) -> np.ndarray:
    """[..., R*32, C*32] -> [..., nnz, 32, 32] in row-major block order (layout.py:40-45)."""
    pos = sparse_positions(pattern)
    out = np.empty(x.shape[:-2] + (len(pos), BLOCK, BLOCK), dtype=x.dtype)
    for k, (i, j) in enumerate(pos):
        out[..., k, :, :] = x[..., i * BLOCK:(i + 1) * BLOCK, j * BLOCK:(j + 1) * BLOCK]
    return out


def to_dense(pattern, x: np.ndarray, fill=0.0) -> np.ndarray:
    """[..., nnz, 32, 32] -> [..., R*32, C*32] (layout.py:47-57).  Absent blocks
    hold ``fill`` (0 for matmul operands, -inf for softmax scores); the
    reference leaves them uninitialised."""
    mask = _as_mask(pattern)
    pos = sparse_positions(pattern)
    out = np.full(x.shape[:-3] + (mask.shape[0] * BLOCK, mask.shape[1] * BLOCK), fill,
                  dtype=x.dtype)
    for k, (i, j) in enumerate(pos):
        out[..., i * BLOCK:(i + 1) * BLOCK, j * BLOCK:(j + 1) * BLOCK] = x[..., k, :, :]
    return out
