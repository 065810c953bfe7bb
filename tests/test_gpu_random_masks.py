"""GPU: every operator on seeded random masks of odd shapes and densities against the float64 oracles."""
import zlib

import numpy as np
import pytest
import torch

from oracle import attention_oracle as ao, matmul_oracle as mo, softmax_oracle as so
from helpers import operand_shapes, rel_err, to_np

pytestmark = pytest.mark.gpu


def _masks():
    rng = np.random.RandomState(2024)
    out = []
    for i in range(14):
        rows, cols = int(rng.randint(1, 28)), int(rng.randint(1, 28))
        density = float(rng.choice([0.05, 0.2, 0.5, 0.9]))
        m = (rng.rand(rows, cols) < density).astype(np.int64)
        if i % 3 == 0 and m.size > 1:
            m[rng.randint(rows)] = 1                       # one full row: a long group in the row table
        if i % 4 == 1 and m.size > 1:
            m[:, rng.randint(cols)] = 1                    # one full column
        out.append((f"m{i}_{rows}x{cols}_d{density}", m))
    return out


MASKS = _masks()


@pytest.mark.parametrize("name,mask", MASKS, ids=[n for n, _ in MASKS])
def test_matmul_modes(name, mask):
    import sparse
    rng = np.random.RandomState(zlib.crc32(name.encode()))
    L = sparse.SparseLayout(torch.as_tensor(mask))
    for mode in ("sdd", "dsd", "dds"):
        ta, tb = bool(rng.randint(2)), bool(rng.randint(2))
        free = int(rng.choice([32, 64, 96, 128]))
        batch = tuple(int(x) for x in rng.randint(1, 4, size=int(rng.randint(1, 3))))
        sa, sb = operand_shapes(mode, mask, free, ta, tb, batch)
        g = torch.Generator().manual_seed(int(rng.randint(1 << 30)))
        a, b = torch.randn(sa, generator=g).half(), torch.randn(sb, generator=g).half()
        c = sparse.matmul(a.cuda(), b.cuda(), mode, L, ta, tb)
        ref = mo.matmul(to_np(a), to_np(b), mode, mask, ta, tb)
        assert tuple(c.shape) == ref.shape
        if ref.size:
            assert rel_err(to_np(c), ref) <= 2e-3, (mode, ta, tb, free, batch)


@pytest.mark.parametrize("name,mask", MASKS, ids=[n for n, _ in MASKS])
def test_softmax_and_attention(name, mask):
    import sparse
    rng = np.random.RandomState(zlib.crc32(name.encode()) ^ 1)
    L = sparse.SparseLayout(torch.as_tensor(mask))
    rows, cols = mask.shape
    nnz = int(mask.sum())
    causal = bool(rng.randint(2))
    scale = float(rng.choice([0.125, 0.5, 1.0]))
    g = torch.Generator().manual_seed(int(rng.randint(1 << 30)))
    x = (2 * torch.randn(2, nnz, 32, 32, generator=g)).half()
    y = sparse.softmax(x.cuda(), L, scale, causal)
    if nnz:
        assert rel_err(to_np(y), so.forward(to_np(x), mask, scale, causal)) <= 2e-3
    q = torch.randn(2, 32 * rows, 64, generator=g).half().cuda().requires_grad_(True)
    k = torch.randn(2, 32 * cols, 64, generator=g).half().cuda().requires_grad_(True)
    v = torch.randn(2, 32 * cols, 64, generator=g).half().cuda().requires_grad_(True)
    dout = torch.randn(2, 32 * rows, 64, generator=g).half().cuda()
    out = sparse.attention(q, k, v, L, scale, causal)
    qn, kn, vn = (to_np(t.detach()) for t in (q, k, v))
    ref = ao.forward(qn, kn, vn, mask, scale, causal)
    assert torch.isfinite(out).all()
    assert rel_err(to_np(out.detach()), ref) <= 2e-3
    out.backward(dout)
    for got, want in zip((q.grad, k.grad, v.grad), ao.backward(qn, kn, vn, to_np(dout), mask, scale, causal)):
        assert torch.isfinite(got).all()
        assert rel_err(to_np(got), want) <= 8e-3
