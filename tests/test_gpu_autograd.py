"""GPU: gradients of sparse.matmul / sparse.softmax against the oracle's matrix calculus."""
import itertools

import numpy as np
import pytest
import torch

from oracle import matmul_oracle as mo, softmax_oracle as so
from helpers import mask_zoo, operand_shapes, rel_err, to_np, tol_of

pytestmark = pytest.mark.gpu
ZOO = dict(mask_zoo())
VARIANTS = list(itertools.product(("sdd", "dsd", "dds"), (False, True), (False, True)))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("mode,ta,tb", VARIANTS)
def test_matmul_backward_all_variants(mode, ta, tb, dtype):
    """All 12 forward variants; their backward calls exercise the transposed walks."""
    import sparse
    mask = np.asarray(ZOO["empty_row_col_6x5"])
    g = torch.Generator().manual_seed(3)
    sa, sb = operand_shapes(mode, mask, 64, ta, tb, (2,))
    a = torch.randn(sa, generator=g).to(dtype)
    b = torch.randn(sb, generator=g).to(dtype)
    L = sparse.SparseLayout(torch.as_tensor(mask))
    ad, bd = a.cuda().requires_grad_(True), b.cuda().requires_grad_(True)
    c = sparse.matmul(ad, bd, mode, L, ta, tb)
    dc = torch.randn(c.shape, generator=g).to(dtype)
    c.backward(dc.cuda())
    da, db = mo.backward_dense(to_np(a), to_np(b), to_np(dc), mode, mask, ta, tb)
    assert ad.grad.shape == a.shape and bd.grad.shape == b.shape
    assert rel_err(to_np(ad.grad), da) <= tol_of(dtype)
    assert rel_err(to_np(bd.grad), db) <= tol_of(dtype)


def test_attention_chain_gradients_fp32():
    """q, k, v gradients of softmax(q k^T / 8) v on a block mask against dense torch autograd."""
    import sparse
    mask = torch.as_tensor(np.asarray(ZOO["rand16"]))
    L = sparse.SparseLayout(mask)
    g = torch.Generator().manual_seed(4)
    q, k, v = (torch.randn(2, 512, 64, generator=g) for _ in range(3))
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    s = sparse.matmul(qd, kd, "sdd", L, False, True)
    p = sparse.softmax(s, L, 0.125, False)
    o = sparse.matmul(p, vd, "dsd", L)
    do = torch.randn(o.shape, generator=g)
    o.backward(do.cuda())

    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    big = mask.repeat_interleave(32, 0).repeat_interleave(32, 1).bool()
    sc = (qr @ kr.transpose(-1, -2)) * 0.125
    pr = torch.softmax(sc.masked_fill(~big, float("-inf")), -1)
    (pr @ vr).backward(do.double())
    assert rel_err(to_np(o), (pr @ vr).detach().numpy()) <= 1e-5
    for got, ref in ((qd, qr), (kd, kr), (vd, vr)):
        assert rel_err(to_np(got.grad), ref.grad.numpy()) <= 2e-5


def test_needs_input_grad_is_respected():
    import sparse
    mask = torch.as_tensor(np.asarray(ZOO["known3x3"]))
    L = sparse.SparseLayout(mask)
    a = torch.randn(1, 96, 64, device="cuda", requires_grad=True)
    b = torch.randn(1, 96, 64, device="cuda")
    sparse.matmul(a, b, "sdd", L, False, True).sum().backward()
    assert a.grad is not None and b.grad is None
