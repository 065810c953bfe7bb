"""CPU: the dense matmul oracle against the C block walk, library GEMMs and matrix calculus."""
import itertools

import numpy as np
import pytest

from oracle import c_oracle, layout_oracle as lo, matmul_oracle as mo
from helpers import mask_zoo, operand_shapes

SMALL = [(n, m) for n, m in mask_zoo() if n in ("known3x3", "single", "empty_row_col_6x5", "tall_7x2", "wide_2x9")]
VARIANTS = list(itertools.product(("sdd", "dsd", "dds"), (False, True), (False, True)))


def _operands(mode, mask, free, ta, tb, seed=0, batch=(2,)):
    rng = np.random.RandomState(seed)
    sa, sb = operand_shapes(mode, mask, free, ta, tb, batch)
    return rng.randn(*sa).astype(np.float32), rng.randn(*sb).astype(np.float32)


@pytest.mark.parametrize("name,mask", SMALL)
@pytest.mark.parametrize("mode,ta,tb", VARIANTS)
def test_dense_meaning_equals_block_walk(name, mask, mode, ta, tb):
    """Two independent restatements (dense algebra in numpy, table walk in C) agree."""
    mask = np.asarray(mask)
    a, b = _operands(mode, mask, 64, ta, tb)
    ref = mo.matmul(a, b, mode, mask, ta, tb)
    walk = c_oracle.matmul(a, b, mode, mask, ta, tb)
    assert ref.shape == walk.shape
    assert mo.rel_err(walk, ref) < 1e-12


def test_full_mask_reduces_to_plain_gemm():
    mask = np.ones((3, 2), dtype=np.int64)
    rng = np.random.RandomState(1)
    a = rng.randn(2, 96, 40)
    b = rng.randn(2, 40, 64)
    c = mo.matmul(a, b, "sdd", mask)                      # to_sparse(a @ b)
    assert np.allclose(lo.to_dense(mask, c), a @ b, rtol=0, atol=1e-12)
    s = lo.to_sparse(mask, rng.randn(2, 96, 64))
    d = rng.randn(2, 64, 32)
    assert np.allclose(mo.matmul(s, d, "dsd", mask), lo.to_dense(mask, s) @ d, atol=1e-12)
    e = rng.randn(2, 32, 96)
    assert np.allclose(mo.matmul(e, s, "dds", mask), e @ lo.to_dense(mask, s), atol=1e-12)


def test_identity_blocks_gather_rows():
    """With identity blocks a DSD copies the dense rows each block points at."""
    mask = np.array([[0, 1, 0], [1, 0, 1]])
    s = np.broadcast_to(np.eye(32), (1, 3, 32, 32)).copy()
    b = np.random.RandomState(2).randn(1, 96, 32)
    c = mo.matmul(s, b, "dsd", mask)
    assert np.allclose(c[0, :32], b[0, 32:64])
    assert np.allclose(c[0, 32:], b[0, :32] + b[0, 64:])
    # transposed sparse operand: column groups, contraction over block rows
    ct = mo.matmul(s, np.random.RandomState(3).randn(1, 64, 32), "dsd", mask, True, False)
    assert ct.shape == (1, 96, 32)


def test_transposes_are_transposes():
    mask = np.asarray(dict(mask_zoo())["empty_row_col_6x5"])
    rng = np.random.RandomState(4)
    a = rng.randn(1, 6 * 32, 64)
    b = rng.randn(1, 64, 5 * 32)
    base = mo.matmul(a, b, "sdd", mask)
    assert np.array_equal(mo.matmul(a.swapaxes(-1, -2).copy(), b, "sdd", mask, True, False), base)
    assert np.array_equal(mo.matmul(a, b.swapaxes(-1, -2).copy(), "sdd", mask, False, True), base)
    # (S^T) B == (B^T S)^T
    s = rng.randn(1, int(mask.sum()), 32, 32)
    d = rng.randn(1, 6 * 32, 64)
    lhs = mo.matmul(s, d, "dsd", mask, True, False)
    rhs = mo.matmul(d.swapaxes(-1, -2).copy(), s, "dds", mask, False, False).swapaxes(-1, -2)
    assert np.allclose(lhs, rhs, atol=1e-12)


@pytest.mark.parametrize("mode,ta,tb", VARIANTS)
def test_backward_plan_matches_matrix_calculus(mode, ta, tb):
    """The mode/transposition algebra of the backward gives the gradients of the dense meaning."""
    mask = np.asarray(dict(mask_zoo())["empty_row_col_6x5"])
    a, b = _operands(mode, mask, 32, ta, tb, seed=5, batch=(1,))
    c = mo.matmul(a, b, mode, mask, ta, tb)
    dc = np.random.RandomState(6).randn(*c.shape)
    da1, db1 = mo.backward(a, b, dc, mode, mask, ta, tb)
    da2, db2 = mo.backward_dense(a, b, dc, mode, mask, ta, tb)
    assert da1.shape == a.shape and db1.shape == b.shape
    assert mo.rel_err(da1, da2) < 1e-12 and mo.rel_err(db1, db2) < 1e-12


def test_backward_by_finite_differences():
    mask = np.array([[1, 0], [1, 1]])
    rng = np.random.RandomState(8)
    a = rng.randn(1, 64, 32)
    b = rng.randn(1, 64, 32)
    dc = rng.randn(1, 3, 32, 32)
    da, db = mo.backward(a, b, dc, "sdd", mask, False, True)
    f = lambda a_, b_: float(np.sum(mo.matmul(a_, b_, "sdd", mask, False, True) * dc))
    eps = 1e-6
    for (i, j) in ((0, 0), (37, 5), (63, 31)):
        ap = a.copy(); ap[0, i, j] += eps
        am = a.copy(); am[0, i, j] -= eps
        assert abs((f(ap, b) - f(am, b)) / (2 * eps) - da[0, i, j]) < 1e-5
        bp = b.copy(); bp[0, i, j] += eps
        bm = b.copy(); bm[0, i, j] -= eps
        assert abs((f(a, bp) - f(a, bm)) / (2 * eps) - db[0, i, j]) < 1e-5
