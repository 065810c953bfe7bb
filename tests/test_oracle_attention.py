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


# ---- backward ------------------------------------------------------------------------------------

@pytest.mark.parametrize("name,causal", [("known3x3", False), ("known3x3", True), ("empty_row_col_6x5", False), ("rand16", True)])
def test_backward_equals_the_chain_of_stage_backwards(name, causal):
    """dq, dk, dv through the three stage oracles (SDD, softmax, DSD and their backward functions)."""
    mask = np.asarray(ZOO[name])
    q, k, v = _qkv(mask, d=16, seed=11)
    dout = np.random.RandomState(12).randn(*q.shape)
    s = mo.matmul(q, k, "sdd", mask, False, True)
    p = so.forward(s, mask, 0.2, causal)
    dp, dv = mo.backward(p, v, dout, "dsd", mask)
    ds = so.backward(p, dp, mask, 0.2)
    dq, dk = mo.backward(q, k, ds, "sdd", mask, False, True)
    for got, want in zip(ao.backward(q, k, v, dout, mask, 0.2, causal), (dq, dk, dv)):
        assert got.shape == want.shape
        assert np.max(np.abs(got - want)) <= 1e-11 * max(1.0, np.max(np.abs(want)))


def test_backward_by_finite_differences():
    """Central differences of sum(forward * dout) along random directions of q, k and v."""
    mask = np.asarray(ZOO["known3x3"])
    q, k, v = _qkv(mask, d=8, batch=(1,), seed=21)
    rng = np.random.RandomState(22)
    dout = rng.randn(*q.shape)
    grads = ao.backward(q, k, v, dout, mask, 0.3, True)
    loss = lambda a, b, c: float(np.sum(ao.forward(a, b, c, mask, 0.3, True) * dout))
    eps = 1e-5
    for i, g in enumerate(grads):
        for _ in range(3):
            d = rng.randn(*g.shape)
            args_p, args_m = [q, k, v], [q, k, v]
            args_p[i] = args_p[i] + eps * d
            args_m[i] = args_m[i] - eps * d
            numeric = (loss(*args_p) - loss(*args_m)) / (2 * eps)
            assert abs(numeric - float(np.sum(g * d))) <= 1e-6 * max(1.0, abs(numeric))


def test_backward_against_torch_autograd_on_the_dense_meaning():
    import torch
    mask = np.asarray(ZOO["rand16"])
    q, k, v = _qkv(mask, d=8, batch=(1,), seed=31)
    dout = np.random.RandomState(32).randn(*q.shape)
    tq, tk, tv = (torch.tensor(t, dtype=torch.float64, requires_grad=True) for t in (q, k, v))
    vis = torch.as_tensor(mask != 0).repeat_interleave(32, 0).repeat_interleave(32, 1)
    vis = vis & torch.ones(vis.shape, dtype=torch.bool).tril()
    s = (0.4 * tq @ tk.transpose(-1, -2)).masked_fill(~vis, float("-inf"))
    w = torch.softmax(s, -1)
    w = torch.where(vis.any(-1, keepdim=True), w, torch.zeros_like(w))
    (w @ tv).backward(torch.tensor(dout))
    for got, want in zip(ao.backward(q, k, v, dout, mask, 0.4, True), (tq.grad, tk.grad, tv.grad)):
        assert np.allclose(got, want.numpy(), atol=1e-10)


def test_backward_rows_and_columns_without_blocks_get_zero_gradients():
    mask = np.asarray(ZOO["empty_row_col_6x5"])
    q, k, v = _qkv(mask, d=8, batch=(1,), seed=41)
    dq, dk, dv = ao.backward(q, k, v, np.ones_like(q), mask, 1.0, False)
    empty_rows = np.repeat(~mask.any(axis=1), 32)
    empty_cols = np.repeat(~mask.any(axis=0), 32)
    assert empty_rows.any() and empty_cols.any()
    assert np.all(dq[0, empty_rows] == 0) and np.all(dk[0, empty_cols] == 0) and np.all(dv[0, empty_cols] == 0)
