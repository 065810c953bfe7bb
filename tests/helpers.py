"""Shared test helpers: mask zoo, tolerances, conversions."""
import numpy as np
import torch

from oracle import layout_oracle as lo

# tolerances of the parity bar: max|out - ref| / max|ref|
TOL_F32 = 1e-5
TOL_F16 = 2e-3


def tol_of(dtype) -> float:
    return TOL_F32 if dtype in (torch.float32, np.float32) else TOL_F16


def mask_zoo():
    """(name, mask) pairs covering the edge cases: empty rows/columns, single block,
    full mask, non-square, wide (256 block columns), random."""
    rng = np.random.RandomState(7)
    zoo = []
    zoo.append(("known3x3", np.array([[1, 0, 1], [0, 1, 0], [1, 1, 0]])))
    zoo.append(("single", np.array([[0, 0], [0, 1]])))
    zoo.append(("one_cell", np.array([[1]])))
    zoo.append(("full4", np.ones((4, 4), dtype=np.int64)))
    m = (rng.rand(6, 5) < 0.4).astype(np.int64)
    m[2, :] = 0
    m[:, 3] = 0
    m[0, 0] = 1
    zoo.append(("empty_row_col_6x5", m))
    zoo.append(("tall_7x2", (rng.rand(7, 2) < 0.6).astype(np.int64) | np.eye(7, 2, dtype=np.int64)))
    zoo.append(("wide_2x9", (rng.rand(2, 9) < 0.5).astype(np.int64) | np.eye(2, 9, dtype=np.int64)))
    zoo.append(("rand16", (rng.rand(16, 16) < 0.3).astype(np.int64) | np.eye(16, dtype=np.int64)))
    long_row = np.zeros((5, 40), dtype=np.int64)
    long_row[1, :] = 1          # one row of 40 blocks: longer than one team's default span
    long_row[3, ::7] = 1
    long_row[:, 2] = 1
    zoo.append(("long_row_5x40", long_row))
    long_col = np.zeros((70, 3), dtype=np.int64)
    long_col[:, 1] = 1          # one column of 70 blocks: cut into parts that meet in the workspace
    long_col[::9, 0] = 1
    long_col[5, 2] = 1
    zoo.append(("long_col_70x3", long_col))
    return zoo


def to_np(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().double().numpy()


def rel_err(out, ref) -> float:
    out = np.asarray(out, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    if ref.size == 0:
        return 0.0
    denom = float(np.max(np.abs(ref)))
    return float(np.max(np.abs(out - ref))) / (denom if denom > 0 else 1.0)


def local_err(out, ref, floor: float = 1e-3) -> float:
    """Largest error of any output row and of any 32 x 32 output tile, each normalised by its OWN largest
    reference value (not less than ``floor`` times the global one, so that rows and tiles that are zero
    or nearly so are held to an absolute bar).  A mistake confined to rows or blocks of small magnitude
    passes ``rel_err`` and fails here.  Works on dense results ``[..., M, N]`` and on block stacks
    ``[..., nnz, 32, 32]`` alike (the last two axes are tiled)."""
    out = np.asarray(out, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    if ref.size == 0:
        return 0.0
    top = float(np.max(np.abs(ref)))
    low = floor * (top if top > 0 else 1.0)
    diff = np.abs(out - ref)
    rows = diff.max(axis=-1) / np.maximum(np.abs(ref).max(axis=-1), low)
    worst = float(rows.max())
    m, n = ref.shape[-2:]
    if m % 32 == 0 and n % 32 == 0:
        tiled = lambda x: x.reshape(x.shape[:-2] + (m // 32, 32, n // 32, 32)).max(axis=(-3, -1))
        worst = max(worst, float((tiled(diff) / np.maximum(tiled(np.abs(ref)), low)).max()))
    return worst


def operand_shapes(mode, mask, free, trans_a, trans_b, batch=(2,)):
    """Stored shapes of a and b for a product on `mask` with free dense dim `free`."""
    R, C = mask.shape
    nnz = int(np.count_nonzero(mask))
    SR, SC = R * lo.BLOCK, C * lo.BLOCK
    sparse = batch + (nnz, lo.BLOCK, lo.BLOCK)
    if mode == "sdd":      # op(a): SR x K, op(b): K x SC
        a = (free, SR) if trans_a else (SR, free)
        b = (SC, free) if trans_b else (free, SC)
        return batch + a, batch + b
    if mode == "dsd":      # op(S): (SR x SC) or transposed; op(b): K x N
        K = SR if trans_a else SC
        b = (free, K) if trans_b else (K, free)
        return sparse, batch + b
    # dds: op(a): M x K; op(S): K x N
    K = SC if trans_b else SR
    a = (K, free) if trans_a else (free, K)
    return batch + a, sparse
