"""Block-sparse row softmax, forward and backward, in float64 (CPU oracle).

TEST INFRASTRUCTURE ONLY: nothing shipped imports this file.

Forward follows the formula of ``sparse_softmax.cu:130-153`` (row max over the
stored blocks of the block row, ``exp(x - max)``, divide by the row sum) with
the two additions this build defines: the scores are multiplied by ``scale``
first, and with ``causal`` every position whose global column exceeds its
global row counts as ``-inf``.  Written as dense algebra:

    y = to_sparse(softmax(scale * dense_neginf(x) + causal_mask, axis=-1))

A row with no finite entry (everything masked) yields zeros, not NaN.

Backward follows ``sparse_softmax.cu:190-203``:
``dx = scale * (dy - sum(dy * y)) * y`` over the stored blocks of the row
(the reference has no scale, i.e. scale = 1).

:func:`forward_blockwalk` recomputes the forward by walking the row table the
way the kernel does; the tests require it to agree with the dense form.
"""
import numpy as np

from . import layout_oracle as lo

BLOCK = lo.BLOCK


def forward(x, pattern, scale: float = 1.0, causal: bool = False):
    x = np.asarray(x, dtype=np.float64)
    dense = lo.to_dense(pattern, x * scale, -np.inf)
    n_rows, n_cols = dense.shape[-2:]
    if causal:
        r = np.arange(n_rows)[:, None]
        c = np.arange(n_cols)[None, :]
        dense = np.where(c > r, -np.inf, dense)
    m = np.max(dense, axis=-1, keepdims=True)
    m = np.where(np.isfinite(m), m, 0.0)
    e = np.exp(dense - m)
    s = np.sum(e, axis=-1, keepdims=True)
    y = np.where(s > 0, e / np.where(s > 0, s, 1.0), 0.0)
    return lo.to_sparse(pattern, y)


def forward_blockwalk(x, pattern, scale: float = 1.0, causal: bool = False):
    """Same result from the row table: per block row, per element row, loop the
    group's blocks (three passes as in sparse_softmax.cu:130-153)."""
    x = np.asarray(x, dtype=np.float64)
    blocks, offsets = lo.create_layout(pattern)
    idx, brow, bcol = lo.decode_blocks(blocks)
    flat = x.reshape((-1,) + x.shape[-3:])
    out = np.zeros_like(flat)
    for b in range(flat.shape[0]):
        for g in range(len(offsets) - 1):
            lo_, hi_ = offsets[g], offsets[g + 1]
            for r in range(BLOCK):
                row_global = g * BLOCK + r
                vals = []
                for p in range(lo_, hi_):
                    v = flat[b, idx[p], r, :] * scale
                    if causal:
                        cols = bcol[p] * BLOCK + np.arange(BLOCK)
                        v = np.where(cols > row_global, -np.inf, v)
                    vals.append(v)
                if not vals:
                    continue
                vals = np.stack(vals)
                m = vals.max()
                if not np.isfinite(m):
                    continue
                e = np.exp(vals - m)
                e /= e.sum()
                for k, p in enumerate(range(lo_, hi_)):
                    out[b, idx[p], r, :] = e[k]
    return out.reshape(x.shape)


def backward(y, dy, pattern, scale: float = 1.0):
    y = np.asarray(y, dtype=np.float64)
    dy = np.asarray(dy, dtype=np.float64)
    yd = lo.to_dense(pattern, y, 0.0)
    dyd = lo.to_dense(pattern, dy, 0.0)
    dot = np.sum(yd * dyd, axis=-1, keepdims=True)
    dx = scale * (dyd - dot) * yd
    return lo.to_sparse(pattern, dx)
