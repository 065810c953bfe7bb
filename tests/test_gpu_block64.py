"""Masks of 64x64 blocks (``SparseLayout(pattern, block=64)``): the reference has 32x32x32 kernels
only (sparse_smm_gpu.cu:22, :106, :192), so the meaning is fixed by the dense definition: every kept
64x64 block is dense, everything else is absent.  The layout runs such a block as its 2x2 tiles of
32x32, so tables and block stack must be those of the mask with every cell repeated twice along both
axes, bit for bit, and every operator must agree with its oracle on that expanded mask."""
import numpy as np
import pytest
import torch

from oracle import attention_oracle as ao
from oracle import layout_oracle as lo
from oracle import matmul_oracle as mo
from oracle import softmax_oracle as so

pytestmark = pytest.mark.gpu

FP16_TOL = 2e-3


def _masks():
    rng = np.random.RandomState(64)
    rand = ((rng.rand(8, 8) < 0.4) | np.eye(8, dtype=bool)).astype(np.int64)
    i, j = np.indices((16, 16))
    causal = ((j <= i) & ((i - j < 2) | (j % 4 == 0))).astype(np.int64)
    ragged = (rng.rand(5, 9) < 0.5).astype(np.int64)
    ragged[2] = 0                                   # an empty block row
    return [("rand8", rand), ("causal16", causal), ("ragged5x9", ragged)]


def _expand(mask):
    return np.kron(mask, np.ones((2, 2), dtype=mask.dtype))


@pytest.mark.parametrize("name,mask", _masks())
def test_tables_are_those_of_the_expanded_mask(name, mask):
    import sparse
    L = sparse.SparseLayout(torch.as_tensor(mask), block=64)
    tiles = _expand(mask)
    assert L.block == 64 and L.tile_shape == tiles.shape and L.num_blocks == 4 * int(mask.sum())
    for tr, got in ((False, L.row_layout), (True, L.col_layout)):
        blocks, offs = lo.create_layout(tiles, tr)
        assert np.array_equal(got[0].cpu().numpy(), blocks) and np.array_equal(got[1].cpu().numpy(), offs)
    g = torch.Generator().manual_seed(7)
    x = torch.randn(2, 64 * mask.shape[0], 64 * mask.shape[1], generator=g).half()
    s = L.to_sparse(x.cuda())
    assert tuple(s.shape) == (2, L.num_blocks, 32, 32)
    kept = torch.as_tensor(np.kron(mask, np.ones((64, 64), dtype=mask.dtype))).bool()
    assert torch.equal(L.to_dense(s).cpu(), x * kept)
    with pytest.raises(ValueError):
        L.to_sparse(x[..., :-32, :].cuda())


@pytest.mark.parametrize("name,mask", _masks()[:2])
def test_operators_on_64_blocks(name, mask):
    import sparse
    L = sparse.SparseLayout(torch.as_tensor(mask), block=64)
    tiles = _expand(mask)
    n = 64 * mask.shape[0]
    g = torch.Generator().manual_seed(n)
    q, k, v = (torch.randn(3, n, 64, generator=g).half() for _ in range(3))
    s = sparse.matmul(q.cuda(), k.cuda(), "sdd", L, False, True)
    ref_s = mo.matmul(q.numpy(), k.numpy(), "sdd", tiles, False, True)
    assert mo.rel_err(s.float().cpu().numpy(), ref_s) <= FP16_TOL
    p = sparse.softmax(s, L, 0.125, True)
    ref_p = so.forward(s.float().cpu().numpy(), tiles, 0.125, True)
    assert mo.rel_err(p.float().cpu().numpy(), ref_p) <= FP16_TOL
    o = sparse.matmul(p, v.cuda(), "dsd", L)
    assert mo.rel_err(o.float().cpu().numpy(), mo.matmul(p.float().cpu().numpy(), v.numpy(), "dsd", tiles)) <= FP16_TOL
    w = sparse.matmul(v.cuda(), p, "dds", L, True, False)
    assert mo.rel_err(w.float().cpu().numpy(),
                      mo.matmul(v.numpy(), p.float().cpu().numpy(), "dds", tiles, True, False)) <= FP16_TOL
    fused = sparse.attention(q.cuda(), k.cuda(), v.cuda(), L, 0.125, True)
    assert mo.rel_err(fused.float().cpu().numpy(), ao.forward(q.numpy(), k.numpy(), v.numpy(), tiles, 0.125, True)) <= FP16_TOL


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("name,mask", _masks() + [("long_rows_3x40", np.ones((3, 40), dtype=np.int64))])
def test_dsd_kernel_that_owns_whole_blocks(name, mask, dtype):
    """The untransposed DSD product on a block=64 layout goes to bsa_matmul_dsd_block64 (a wavefront owns
    64 x 64 blocks, one dense strip serves the upper and the lower tiles): against the oracle on the
    expanded mask, against the walk over 32 x 32 tiles of the same layout, with one sparse operand shared
    by the batch, and with a dense width of 128."""
    import sparse
    from sparse import _ops
    L = sparse.SparseLayout(torch.as_tensor(mask), block=64)
    assert L.coarse_row_layout is not None and L.coarse_row_layout[0].numel() == 2 * int(mask.sum())
    tiles = _expand(mask)
    g = torch.Generator().manual_seed(64 + mask.shape[1])
    tol = FP16_TOL if dtype == torch.float16 else 1e-2
    for width, batch in ((64, 3), (128, 2)):
        s = torch.rand(batch, L.num_blocks, 32, 32, generator=g).to(dtype)
        v = torch.randn(batch, 64 * mask.shape[1], width, generator=g).to(dtype)
        ref = mo.matmul(s.float().numpy().astype(np.float64), v.float().numpy().astype(np.float64), "dsd", tiles)
        calls = []
        real = sparse.kernel.lib.bsa_matmul_dsd_block64
        _ops.USE_BLOCK64_KERNEL = True
        try:
            sparse.kernel.lib.bsa_matmul_dsd_block64 = lambda *a: (calls.append(1), real(*a))[1]
            out = sparse.matmul(s.cuda(), v.cuda(), "dsd", L)
        finally:
            sparse.kernel.lib.bsa_matmul_dsd_block64 = real
            _ops.USE_BLOCK64_KERNEL = False
        assert calls, "the 64 x 64 kernel was not taken"
        assert mo.rel_err(out.float().cpu().numpy(), ref) <= tol
        by_tiles = sparse.matmul(s.cuda(), v.cuda(), "dsd", L)
        assert mo.rel_err(out.float().cpu().numpy(), by_tiles.float().cpu().numpy().astype(np.float64)) <= tol
    # one sparse operand for the whole batch
    s1 = torch.rand(L.num_blocks, 32, 32, generator=g).to(dtype)
    v = torch.randn(2, 64 * mask.shape[1], 64, generator=g).to(dtype)
    _ops.USE_BLOCK64_KERNEL = True
    try:
        out = sparse.matmul(s1.cuda(), v.cuda(), "dsd", L)
    finally:
        _ops.USE_BLOCK64_KERNEL = False
    ref = mo.matmul(s1.expand(2, -1, -1, -1).float().numpy().astype(np.float64), v.float().numpy().astype(np.float64), "dsd", tiles)
    assert mo.rel_err(out.float().cpu().numpy(), ref) <= tol
    # gradients still flow (the backward products take the tile walks)
    sd = torch.rand(1, L.num_blocks, 32, 32, generator=g).to(dtype).cuda().requires_grad_(True)
    vd = torch.randn(1, 64 * mask.shape[1], 64, generator=g).to(dtype).cuda().requires_grad_(True)
    _ops.USE_BLOCK64_KERNEL = True
    try:
        sparse.matmul(sd, vd, "dsd", L).float().sum().backward()
    finally:
        _ops.USE_BLOCK64_KERNEL = False
    assert sd.grad is not None and vd.grad is not None and torch.isfinite(sd.grad).all() and torch.isfinite(vd.grad).all()
