"""CPU: the attention oracle against the composition of the stage oracles and against mathematics."""
import numpy as np
import pytest
from scipy.special import softmax as scipy_softmax

from oracle import attention_oracle as ao, matmul_oracle as mo, softmax_oracle as so
from helpers import mask_zoo

ZOO = dict(mask_zoo())


def _qkv(mask, d=64, batch=(2,), seed=0):
    rng = np.random.RandomState(seed)
    r, c = np.asarray(mask).shape
    return (rng.randn(*batch, 32 * r, d), rng.randn(*batch, 32 * c, d), rng.randn(*batch, 32 * c, d))


@pytest.mark.parametrize("name", ["known3x3", "single", "empty_row_col_6x5", "wide_2x9", "rand16"])
@pytest.mark.parametrize("scale,causal", [(0.125, False), (0.125, True), (1.0, True)])
def test_equals_the_chain_of_stage_oracles(name, scale, causal):
    mask = np.asarray(ZOO[name])
    q, k, v = _qkv(mask, seed=3)
    s = mo.matmul(q, k, "sdd", mask, False, True)
    p = so.forward(s, mask, scale, causal)
    want = mo.matmul(p, v, "dsd", mask)
    got = ao.forward(q, k, v, mask, scale, causal)
    assert got.shape == want.shape
    assert np.max(np.abs(got - want)) <= 1e-12 * max(1.0, np.max(np.abs(want)))


def test_full_mask_is_textbook_attention():
    mask = np.ones((3, 4), dtype=np.int64)
    q, k, v = _qkv(mask, d=16, seed=1)
    want = scipy_softmax(0.25 * q @ np.swapaxes(k, -1, -2), axis=-1) @ v
    assert np.allclose(ao.forward(q, k, v, mask, 0.25, False), want, atol=1e-12)
    sq = np.ones((3, 3), dtype=np.int64)
    q, k, v = _qkv(sq, d=16, seed=2)
    s = 0.25 * q @ np.swapaxes(k, -1, -2)
    s = np.where(np.tril(np.ones((96, 96), dtype=bool)), s, -np.inf)
    assert np.allclose(ao.forward(q, k, v, sq, 0.25, True), scipy_softmax(s, axis=-1) @ v, atol=1e-12)


def test_invariants():
    mask = np.asarray(ZOO["rand16"])
    q, k, v = _qkv(mask, d=8, batch=(1,), seed=5)
    out = ao.forward(q, k, v, mask, 0.3, False)
    # values all ones -> every row that sees anything returns ones (the weights sum to one)
    ones = ao.forward(q, k, np.ones_like(v), mask, 0.3, False)
    seen = np.repeat(mask.any(axis=1), 32)
    assert np.allclose(ones[0, seen], 1.0) and np.all(ones[0, ~seen] == 0.0)
    # permuting keys and values inside one block column changes nothing
    perm = np.arange(k.shape[-2])
    perm[32:64] = perm[32:64][::-1]
    assert np.allclose(ao.forward(q, k[:, perm], v[:, perm], mask, 0.3, False), out, atol=1e-12)
    # a hidden block column has no influence
    c = int(np.argmin(mask.sum(axis=0)))
    hidden = mask.copy()
    hidden[:, c] = 0
    k2, v2 = k.copy(), v.copy()
    k2[:, 32 * c: 32 * c + 32] += 7.0
    v2[:, 32 * c: 32 * c + 32] -= 3.0
    assert np.allclose(ao.forward(q, k2, v2, hidden, 0.3, False), ao.forward(q, k, v, hidden, 0.3, False))
