"""CPU: the softmax oracle against scipy, the table walks and its invariants."""
import numpy as np
import pytest
from scipy.special import softmax as scipy_softmax

from oracle import c_oracle, layout_oracle as lo, softmax_oracle as so
from helpers import mask_zoo

SMALL = [(n, m) for n, m in mask_zoo() if n in ("known3x3", "single", "empty_row_col_6x5", "wide_2x9", "full4")]


@pytest.mark.parametrize("name,mask", SMALL)
@pytest.mark.parametrize("scale,causal", [(1.0, False), (0.125, True), (2.0, True)])
def test_three_restatements_agree(name, mask, scale, causal):
    mask = np.asarray(mask)
    x = (3 * np.random.RandomState(0).randn(2, int(np.count_nonzero(mask)), 32, 32)).astype(np.float32)
    y = so.forward(x, mask, scale, causal)
    assert np.allclose(so.forward_blockwalk(x, mask, scale, causal), y, atol=1e-13)
    assert np.allclose(c_oracle.softmax_fwd(x, mask, scale, causal), y, atol=1e-13)


def test_full_mask_is_plain_softmax():
    mask = np.ones((2, 3), dtype=np.int64)
    x = np.random.RandomState(1).randn(1, 6, 32, 32)
    y = lo.to_dense(mask, so.forward(x, mask, 0.5, False))
    assert np.allclose(y, scipy_softmax(0.5 * lo.to_dense(mask, x), axis=-1), atol=1e-14)


def test_causal_full_mask_is_tril_softmax():
    mask = np.ones((2, 2), dtype=np.int64)
    x = np.random.RandomState(2).randn(1, 4, 32, 32)
    d = lo.to_dense(mask, x)
    d = np.where(np.triu(np.ones((64, 64)), 1) > 0, -np.inf, d)
    y = lo.to_dense(mask, so.forward(x, mask, 1.0, True))
    assert np.allclose(y, scipy_softmax(d, axis=-1), atol=1e-14)
    assert np.all(y[0][np.triu_indices(64, 1)] == 0)


@pytest.mark.parametrize("name,mask", SMALL)
def test_invariants(name, mask):
    mask = np.asarray(mask)
    x = np.random.RandomState(3).randn(1, int(np.count_nonzero(mask)), 32, 32) * 4
    y = so.forward(x, mask, 0.3, False)
    assert np.all(y >= 0) and np.all(y <= 1)
    rows = lo.to_dense(mask, y).sum(-1)[0]
    has_block = np.repeat(mask.sum(1) > 0, 32)
    assert np.allclose(rows[has_block], 1.0, atol=1e-12) and np.all(rows[~has_block] == 0)
    # shift invariance per row
    assert np.allclose(so.forward(x + 7.5, mask, 0.3, False), y, atol=1e-12)
    # huge logits stay finite
    assert np.all(np.isfinite(so.forward(x * 1e4, mask, 1.0, False)))


def test_fully_masked_rows_give_zeros():
    # block row 0 only holds a block right of the diagonal: every entry is hidden by the causal mask
    mask = np.array([[0, 1], [1, 1]])
    x = np.random.RandomState(4).randn(1, 3, 32, 32)
    for f in (so.forward, so.forward_blockwalk, c_oracle.softmax_fwd):
        y = f(x.astype(np.float32), mask, 1.0, True)
        assert np.all(np.isfinite(y)) and np.all(y[0, 0] == 0)
        assert np.allclose(lo.to_dense(mask, y)[0, 32:].sum(-1), 1.0)


@pytest.mark.parametrize("scale", [1.0, 0.125])
def test_backward_matches_walk_and_finite_differences(scale):
    mask = np.asarray(dict(mask_zoo())["known3x3"])
    rng = np.random.RandomState(5)
    x = rng.randn(1, 5, 32, 32)
    y = so.forward(x, mask, scale, False)
    dy = rng.randn(*y.shape)
    dx = so.backward(y, dy, mask, scale)
    assert np.allclose(c_oracle.softmax_bwd(y, dy, mask, scale), dx, atol=1e-6)  # C side reads float32
    f = lambda x_: float(np.sum(so.forward(x_, mask, scale, False) * dy))
    eps = 1e-6
    for (k, i, j) in ((0, 0, 0), (2, 17, 9), (4, 31, 31)):
        xp = x.copy(); xp[0, k, i, j] += eps
        xm = x.copy(); xm[0, k, i, j] -= eps
        assert abs((f(xp) - f(xm)) / (2 * eps) - dx[0, k, i, j]) < 1e-6
