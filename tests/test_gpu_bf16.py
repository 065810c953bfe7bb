"""GPU: bfloat16 operands (fp32 accumulation) through every kernel family, against the float64 oracle
on the bf16-rounded inputs.  Tolerance: bf16 keeps 8 bits of mantissa, one rounding of the result is
2^-9 of the value; max|out - ref| / max|ref| <= 1e-2 is written here as the bar for this type."""
import itertools

import numpy as np
import pytest
import torch

from oracle import attention_oracle as ao, layout_oracle as lo, matmul_oracle as mo, softmax_oracle as so
from helpers import mask_zoo, operand_shapes, rel_err, to_np

pytestmark = pytest.mark.gpu
ZOO = dict(mask_zoo())
TOL_BF16 = 1e-2
BF = torch.bfloat16


@pytest.mark.parametrize("mode,ta,tb", list(itertools.product(("sdd", "dsd", "dds"), (False, True), (False, True))))
@pytest.mark.parametrize("name", ["known3x3", "empty_row_col_6x5", "long_col_70x3"])
def test_matmul_all_variants(name, mode, ta, tb):
    import sparse
    mask = np.asarray(ZOO[name])
    g = torch.Generator().manual_seed(11)
    sa, sb = operand_shapes(mode, mask, 64, ta, tb, (2,))
    a, b = torch.randn(sa, generator=g).to(BF), torch.randn(sb, generator=g).to(BF)
    L = sparse.SparseLayout(torch.as_tensor(mask))
    c = sparse.matmul(a.cuda(), b.cuda(), mode, L, ta, tb)
    assert c.dtype == BF
    assert rel_err(to_np(c), mo.matmul(to_np(a), to_np(b), mode, mask, ta, tb)) <= TOL_BF16


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("name", ["known3x3", "rand16", "long_row_5x40"])
def test_softmax_forward_backward(name, causal):
    import sparse
    mask = np.asarray(ZOO[name])
    L = sparse.SparseLayout(torch.as_tensor(mask))
    g = torch.Generator().manual_seed(12)
    x = (2 * torch.randn(2, L.num_blocks, 32, 32, generator=g)).to(BF)
    dy = torch.randn(2, L.num_blocks, 32, 32, generator=g).to(BF)
    xg = x.cuda().requires_grad_(True)
    y = sparse.softmax(xg, L, 0.125, causal)
    assert y.dtype == BF
    assert rel_err(to_np(y), so.forward(to_np(x), mask, 0.125, causal)) <= TOL_BF16
    y.backward(dy.cuda())
    assert rel_err(to_np(xg.grad), so.backward(to_np(y), to_np(dy), mask, 0.125)) <= TOL_BF16


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("name", ["known3x3", "rand16", "long_row_5x40", "empty_row_col_6x5"])
def test_fused_attention(name, causal):
    import sparse
    mask = np.asarray(ZOO[name])
    r, c = mask.shape
    g = torch.Generator().manual_seed(13)
    q = torch.randn(2, 32 * r, 64, generator=g).to(BF)
    k = torch.randn(2, 32 * c, 64, generator=g).to(BF)
    v = torch.randn(2, 32 * c, 64, generator=g).to(BF)
    L = sparse.SparseLayout(torch.as_tensor(mask))
    out = sparse.attention(q.cuda(), k.cuda(), v.cuda(), L, 0.125, causal)
    assert out.dtype == BF
    assert rel_err(to_np(out), ao.forward(to_np(q), to_np(k), to_np(v), mask, 0.125, causal)) <= TOL_BF16


def test_block_copies_and_gradients():
    import sparse
    mask = np.asarray(ZOO["rand16"])
    L = sparse.SparseLayout(torch.as_tensor(mask))
    x = torch.randn(2, 512, 512, generator=torch.Generator().manual_seed(14)).to(BF)
    s = L.to_sparse(x.cuda())
    assert np.array_equal(to_np(s), lo.to_sparse(mask, to_np(x)))
    assert np.array_equal(to_np(L.to_dense(s)), lo.to_dense(mask, lo.to_sparse(mask, to_np(x)), 0.0))
    # one product through autograd in bf16
    a = torch.randn(2, 512, 64).to(BF).cuda().requires_grad_(True)
    b = torch.randn(2, 512, 64).to(BF).cuda().requires_grad_(True)
    sparse.matmul(a, b, "sdd", L, False, True).float().sum().backward()
    assert a.grad.dtype == BF and torch.isfinite(a.grad.float()).all() and torch.isfinite(b.grad.float()).all()
    ga, gb = mo.backward(to_np(a), to_np(b), np.ones((2, L.num_blocks, 32, 32)), "sdd", mask, False, True)
    assert rel_err(to_np(a.grad), ga) <= TOL_BF16 and rel_err(to_np(b.grad), gb) <= TOL_BF16
