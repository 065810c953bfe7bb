"""GPU: every operator on seeded random masks of odd shapes and densities against the float64 oracles."""
import zlib

import numpy as np
import pytest
import torch

from oracle import attention_oracle as ao, matmul_oracle as mo, softmax_oracle as so
from helpers import local_err, operand_shapes, rel_err, to_np

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
            assert local_err(to_np(c), ref) <= 2e-3, (mode, ta, tb, free, batch)


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


@pytest.mark.parametrize("seed", range(10))
def test_groups_around_the_split_boundaries(seed):
    """Rows or columns of 47 to 150 blocks (a group longer than cap * waves pairs is cut into parts that
    meet in a workspace: 40 pairs in the DSD / DDS walks, 48 or 24 in the attention walks), with full rows,
    full columns and empty rows thrown in: the fused attention forward and backward, DSD and DDS."""
    import sparse
    from sparse import _ops
    rng = np.random.RandomState(1000 + seed)
    rows, cols = int(rng.randint(2, 9)), int(rng.choice([47, 48, 49, 65, 96, 97, 130, 150]))
    if seed % 2:
        rows, cols = cols, rows
    mask = (rng.rand(rows, cols) < rng.choice([0.02, 0.1, 0.4])).astype(np.int64)
    for _ in range(int(rng.randint(1, 4))):
        if rng.rand() < 0.5:
            mask[rng.randint(rows), rng.randint(0, max(cols // 3, 1)):] = 1
        else:
            mask[rng.randint(0, max(rows // 3, 1)):, rng.randint(cols)] = 1
    if rng.rand() < 0.3:
        mask[rng.randint(rows)] = 0
    causal, batch = bool(rng.randint(2)), int(rng.randint(1, 4))
    scale = float(rng.choice([0.125, 0.09, 0.5]))
    g = torch.Generator().manual_seed(int(rng.randint(1 << 30)))
    mk = lambda n: (0.7 * torch.randn(batch, 32 * n, 64, generator=g)).half()
    q, k, v, dout = mk(rows), mk(cols), mk(cols), mk(rows)
    L = sparse.SparseLayout(torch.as_tensor(mask))
    rl, cl = L.row_layout, L.col_layout
    qd, kd, vd, dd = (t.cuda() for t in (q, k, v, dout))
    out, lse = _ops.sparse_attention_forward(qd, kd, vd, rl[0], rl[1], scale, causal, cl, return_lse=True)
    assert rel_err(to_np(out), ao.forward(to_np(q), to_np(k), to_np(v), mask, scale, causal)) <= 2e-3
    grads = _ops.sparse_attention_backward(qd, kd, vd, dd, out, lse, rl[0], rl[1], cl[0], cl[1], scale, causal)
    for got, want in zip(grads, ao.backward(to_np(q), to_np(k), to_np(v), to_np(dout), mask, scale, causal)):
        assert rel_err(to_np(got), want) <= 8e-3
    p = sparse.softmax(sparse.matmul(qd, kd, "sdd", L, False, True), L, scale, causal)
    assert rel_err(to_np(sparse.matmul(p, vd, "dsd", L)), mo.matmul(to_np(p), to_np(v), "dsd", mask)) <= 2e-3
    assert rel_err(to_np(sparse.matmul(dd, p, "dds", L, True, False)),
                   mo.matmul(to_np(dout), to_np(p), "dds", mask, True, False)) <= 2e-3
