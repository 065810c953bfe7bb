"""GPU: block-sparse softmax forward / backward against the float64 oracle."""
import numpy as np
import pytest
import torch

from oracle import layout_oracle as lo, softmax_oracle as so
from helpers import mask_zoo, rel_err, to_np, tol_of

pytestmark = pytest.mark.gpu
ZOO = dict(mask_zoo())


def _fwd(mask, dtype, scale, causal, batch=(2,), std=2.0, seed=0):
    import sparse
    mask = np.asarray(mask)
    nnz = int(np.count_nonzero(mask))
    x = (std * torch.randn(batch + (nnz, 32, 32), generator=torch.Generator().manual_seed(seed))).to(dtype)
    L = sparse.SparseLayout(torch.as_tensor(mask))
    y = sparse.softmax(x.cuda(), L, scale, causal)
    ref = so.forward(to_np(x), mask, scale, causal)
    assert y.dtype == dtype and tuple(y.shape) == ref.shape
    return to_np(y), ref


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("scale,causal", [(1.0, False), (0.125, True), (0.125, False), (1.0, True)])
@pytest.mark.parametrize("name", ["known3x3", "single", "one_cell", "full4", "empty_row_col_6x5",
                                  "wide_2x9", "rand16", "long_row_5x40"])
def test_forward(name, scale, causal, dtype):
    y, ref = _fwd(ZOO[name], dtype, scale, causal)
    assert np.all(np.isfinite(y))
    assert rel_err(y, ref) <= tol_of(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_long_rows_take_the_streaming_path(dtype):
    """256 blocks in one row: 32 per wavefront, beyond the register-resident capacity."""
    mask = np.zeros((3, 256), dtype=np.int64)
    mask[0, :] = 1
    mask[1, ::5] = 1
    mask[2, 200:] = 1
    y, ref = _fwd(mask, dtype, 0.125, False, batch=(2,), std=3.0)
    assert rel_err(y, ref) <= tol_of(dtype)
    y, ref = _fwd(mask, dtype, 1.0, True, batch=(1,), std=3.0)
    assert rel_err(y, ref) <= tol_of(dtype)


def test_fully_masked_rows_and_large_logits():
    mask = np.array([[0, 1], [1, 1]])
    y, ref = _fwd(mask, torch.float32, 1.0, True)
    assert np.all(np.isfinite(y)) and np.all(y[:, 0] == 0)
    assert rel_err(y, ref) <= 1e-5
    y, ref = _fwd(ZOO["known3x3"], torch.float32, 1.0, False, std=300.0)
    assert np.all(np.isfinite(y)) and rel_err(y, ref) <= 1e-5
    y, ref = _fwd(ZOO["known3x3"], torch.float16, 1.0, False, std=1000.0)
    assert np.all(np.isfinite(y)) and rel_err(y, ref) <= 2e-3


def test_invariants_on_device():
    import sparse
    mask = np.asarray(ZOO["rand16"])
    L = sparse.SparseLayout(torch.as_tensor(mask))
    x = torch.randn(3, L.num_blocks, 32, 32, device="cuda") * 3
    y = sparse.softmax(x, L, 0.5, False)
    rows = L.to_dense(y).sum(-1)
    assert torch.allclose(rows, torch.ones_like(rows), atol=1e-5)
    assert torch.all(y >= 0) and torch.all(y <= 1)
    assert torch.allclose(sparse.softmax(x + 11.0, L, 0.5, False), y, atol=1e-5)


def test_config3_softmax_fp16():
    import sparse, workloads as wl
    cfg = wl.config3(batch=16)
    L = sparse.SparseLayout(cfg["mask"])
    y = sparse.softmax(cfg["x"].cuda(), L, cfg["scale"], cfg["causal"])
    # oracle on 2 of the 16 heads, invariants on all
    ref = so.forward(to_np(cfg["x"][:2]), cfg["mask"].numpy(), cfg["scale"], cfg["causal"])
    assert rel_err(to_np(y[:2]), ref) <= 2e-3
    rows = L.to_dense(y.float()).sum(-1)
    assert torch.allclose(rows, torch.ones_like(rows), atol=4e-3)
    # strictly-upper part of the diagonal blocks is exactly zero
    dense = L.to_dense(y)
    assert torch.count_nonzero(torch.triu(dense, 1)) == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("name", ["known3x3", "rand16", "long_row_5x40", "empty_row_col_6x5"])
@pytest.mark.parametrize("scale", [1.0, 0.125])
def test_backward(name, scale, dtype):
    import sparse
    mask = np.asarray(ZOO[name])
    L = sparse.SparseLayout(torch.as_tensor(mask))
    g = torch.Generator().manual_seed(1)
    x = (2 * torch.randn(2, L.num_blocks, 32, 32, generator=g)).to(dtype)
    dy = torch.randn(2, L.num_blocks, 32, 32, generator=g).to(dtype)
    xg = x.cuda().requires_grad_(True)
    y = sparse.softmax(xg, L, scale, False)
    y.backward(dy.cuda())
    ref = so.backward(to_np(y), to_np(dy), mask, scale)      # from the y the device produced
    assert rel_err(to_np(xg.grad), ref) <= tol_of(dtype)
    if dtype == torch.float32:                                # and end to end against the oracle forward
        ref2 = so.backward(so.forward(to_np(x), mask, scale, False), to_np(dy), mask, scale)
        assert rel_err(to_np(xg.grad), ref2) <= 1e-5


def test_backward_long_rows():
    import sparse
    mask = np.zeros((2, 256), dtype=np.int64)
    mask[0, :] = 1
    mask[1, ::3] = 1
    L = sparse.SparseLayout(torch.as_tensor(mask))
    g = torch.Generator().manual_seed(2)
    y = torch.rand(1, L.num_blocks, 32, 32, generator=g).half()
    dy = torch.randn(1, L.num_blocks, 32, 32, generator=g).half()
    from sparse.kernel import sparse_ops
    dx = sparse_ops.sparse_softmax_backward(y.cuda(), dy.cuda(), L.row_layout[0], L.row_layout[1], 0.5)
    assert rel_err(to_np(dx), so.backward(to_np(y), to_np(dy), mask, 0.5)) <= 2e-3


def _tri(n):
    return np.tril(np.ones((n, n), dtype=np.int64))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("causal", [False, True])
def test_every_row_length_up_to_50(dtype, causal):
    """Lower-triangular mask: row r has r + 1 blocks, so every specialisation of the register-resident
    walk (1..48 blocks: lanes past the row's end in every position) and the first team rows are hit."""
    y, ref = _fwd(_tri(50), dtype, 0.125, causal, batch=(2,), std=2.0, seed=5)
    assert np.all(np.isfinite(y))
    assert rel_err(y, ref) <= tol_of(dtype)
    rows = y.reshape(2, -1, 32, 32).sum(axis=-1)            # per block: sum over its columns
    offs = lo.create_layout(_tri(50))[1]
    for r in range(50):
        assert np.allclose(rows[:, offs[r]:offs[r + 1]].sum(axis=1), 1.0, atol=5e-3 if dtype == torch.float16 else 1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_backward_every_row_length_up_to_26(dtype):
    import sparse
    from sparse.kernel import sparse_ops
    mask = _tri(26)
    L = sparse.SparseLayout(torch.as_tensor(mask))
    g = torch.Generator().manual_seed(3)
    y = torch.rand(2, L.num_blocks, 32, 32, generator=g).to(dtype)
    dy = torch.randn(2, L.num_blocks, 32, 32, generator=g).to(dtype)
    dx = sparse_ops.sparse_softmax_backward(y.cuda(), dy.cuda(), L.row_layout[0], L.row_layout[1], 0.25)
    assert rel_err(to_np(dx), so.backward(to_np(y), to_np(dy), mask, 0.25)) <= tol_of(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("slice_max,slices", [(64, 2), (64, 4), (64, 8), (5, 4), (5, 2), (5, 8), (-1, 2)])
def test_schedules_the_resident_walk_does_not_take(monkeypatch, dtype, slice_max, slices):
    """Sliced rows longer than the register capacity, or cut into another number of slices than the
    kernel keeps in registers, go through the two-pass walk and give the same result."""
    import sparse
    from sparse import _ops
    from sparse.kernel import sparse_ops
    monkeypatch.setattr(_ops, "SOFTMAX_SLICE_MAX", {torch.float16: (slice_max, slice_max), torch.float32: (slice_max, slice_max)})
    monkeypatch.setattr(_ops, "SOFTMAX_SLICES", {torch.float16: (slices, slices), torch.float32: (slices, slices)})
    mask = np.asarray(ZOO["long_row_5x40"])
    mask = np.concatenate([mask, _tri(40)[:30]], axis=0)
    y, ref = _fwd(mask, dtype, 0.125, True, batch=(2,), std=2.0, seed=9)
    assert rel_err(y, ref) <= tol_of(dtype)
    L = sparse.SparseLayout(torch.as_tensor(mask))
    g = torch.Generator().manual_seed(4)
    yy = torch.rand(2, L.num_blocks, 32, 32, generator=g).to(dtype)
    dy = torch.randn(2, L.num_blocks, 32, 32, generator=g).to(dtype)
    dx = sparse_ops.sparse_softmax_backward(yy.cuda(), dy.cuda(), L.row_layout[0], L.row_layout[1], 0.25)
    assert rel_err(to_np(dx), so.backward(to_np(yy), to_np(dy), mask, 0.25)) <= tol_of(dtype)
