"""GPU: SDD / DSD / DDS through the Python boundary and the C ABI against the dense oracle."""
import itertools

import numpy as np
import pytest
import torch

from oracle import layout_oracle as lo, matmul_oracle as mo
from helpers import local_err, mask_zoo, operand_shapes, rel_err, to_np, tol_of

pytestmark = pytest.mark.gpu

VARIANTS = list(itertools.product(("sdd", "dsd", "dds"), (False, True), (False, True)))
ZOO = dict(mask_zoo())


def _run(mode, mask, free, ta, tb, dtype, batch=(2,), seed=0):
    import sparse
    mask = np.asarray(mask)
    g = torch.Generator().manual_seed(seed)
    sa, sb = operand_shapes(mode, mask, free, ta, tb, batch)
    a = torch.randn(sa, generator=g).to(dtype)
    b = torch.randn(sb, generator=g).to(dtype)
    L = sparse.SparseLayout(torch.as_tensor(mask))
    c = sparse.matmul(a.cuda(), b.cuda(), mode, L, ta, tb)
    ref = mo.matmul(to_np(a), to_np(b), mode, mask, ta, tb)
    assert c.dtype == dtype and tuple(c.shape) == ref.shape
    # the global bar and, at the same tolerance, every output row and every 32 x 32 output tile on its own
    return max(rel_err(to_np(c), ref), local_err(to_np(c), ref))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("mode,ta,tb", VARIANTS)
@pytest.mark.parametrize("name", ["known3x3", "empty_row_col_6x5", "long_row_5x40", "long_col_70x3"])
def test_all_variants(name, mode, ta, tb, dtype):
    err = _run(mode, ZOO[name], 64, ta, tb, dtype)
    assert err <= tol_of(dtype), err


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("mode,ta,tb", VARIANTS)
@pytest.mark.parametrize("free", [32, 96, 128, 160])
def test_free_dimension_sizes(mode, ta, tb, free, dtype):
    err = _run(mode, ZOO["tall_7x2"], free, ta, tb, dtype, batch=(1,), seed=free)
    assert err <= tol_of(dtype), err


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("name", ["single", "one_cell", "full4", "wide_2x9", "rand16"])
@pytest.mark.parametrize("mode", ["sdd", "dsd", "dds"])
def test_edge_layouts(name, mode, dtype):
    for ta, tb in ((False, False), (True, True)):
        err = _run(mode, ZOO[name], 64, ta, tb, dtype, batch=(3,))
        assert err <= tol_of(dtype), (err, ta, tb)


@pytest.mark.parametrize("mode,ta,tb", [("sdd", False, True), ("dsd", False, False), ("dds", True, False)])
def test_multiple_batch_dims_and_many_batches(mode, ta, tb):
    assert _run(mode, ZOO["known3x3"], 64, ta, tb, torch.float16, batch=(2, 3)) <= tol_of(torch.float16)
    assert _run(mode, ZOO["known3x3"], 64, ta, tb, torch.float32, batch=(19,)) <= tol_of(torch.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("mode,ta,tb", [("dsd", False, False), ("dsd", True, False), ("dds", False, False), ("dds", False, True)])
def test_split_groups_reuse_their_workspace(mode, ta, tb, dtype):
    """Groups longer than one workgroup's span are cut into parts that meet in a workspace the
    library leaves zeroed: repeated calls, three 64-wide strips, several batches."""
    import sparse
    from sparse import _ops
    old = _ops.SCHEDULE_GROUP_WALK, _ops.SCHEDULE_GROUP_WALK_LONG
    try:
        for sched in ((2, 2), (4, 8), (3, 1)):
            _ops.SCHEDULE_GROUP_WALK = _ops.SCHEDULE_GROUP_WALK_LONG = sched
            for name in ("long_row_5x40", "long_col_70x3"):
                errs = [_run(mode, ZOO[name], 160, ta, tb, dtype, batch=(3,), seed=s) for s in range(3)]
                assert max(errs) <= tol_of(dtype), (sched, name, errs)
    finally:
        _ops.SCHEDULE_GROUP_WALK, _ops.SCHEDULE_GROUP_WALK_LONG = old


def test_split_result_is_deterministic():
    import sparse
    mask = np.asarray(ZOO["long_col_70x3"])
    L = sparse.SparseLayout(torch.as_tensor(mask))
    g = torch.Generator().manual_seed(5)
    a = torch.randn(4, 64, 70 * 32, generator=g).half().cuda()
    s = torch.randn(4, L.num_blocks, 32, 32, generator=g).half().cuda()
    outs = [sparse.matmul(a, s, "dds", L) for _ in range(5)]
    assert all(torch.equal(outs[0], o) for o in outs[1:])


def test_empty_mask_gives_zeros():
    import sparse
    mask = np.zeros((2, 3), dtype=np.int64)
    L = sparse.SparseLayout(torch.as_tensor(mask))
    s = torch.zeros(2, 0, 32, 32, device="cuda", dtype=torch.float16)
    b = torch.randn(2, 96, 64, device="cuda", dtype=torch.float16)
    c = sparse.matmul(s, b, "dsd", L)
    assert tuple(c.shape) == (2, 64, 64) and torch.count_nonzero(c) == 0
    a = torch.randn(2, 64, 32, device="cuda", dtype=torch.float16)
    d = sparse.matmul(a, b[:, :, :32].contiguous(), "sdd", L, False, True)
    assert tuple(d.shape) == (2, 0, 32, 32)


def test_wide_layout_beyond_256_block_columns():
    """Columns past 255 need the 16-bit decode."""
    import sparse
    mask = np.zeros((2, 300), dtype=np.int64)
    mask[0, 256] = mask[1, 299] = mask[1, 3] = 1
    g = torch.Generator().manual_seed(3)
    s = torch.randn(1, 3, 32, 32, generator=g).half()
    b = torch.randn(1, 300 * 32, 64, generator=g).half()
    L = sparse.SparseLayout(torch.as_tensor(mask))
    c = sparse.matmul(s.cuda(), b.cuda(), "dsd", L)
    assert rel_err(to_np(c), mo.matmul(to_np(s), to_np(b), "dsd", mask)) <= tol_of(torch.float16)


def test_config1_sdd_fp32():
    import sparse, workloads as wl
    cfg = wl.config1()
    L = sparse.SparseLayout(cfg["mask"])
    c = sparse.matmul(cfg["a"].cuda(), cfg["b"].cuda(), "sdd", L, False, True)
    ref = mo.matmul(to_np(cfg["a"]), to_np(cfg["b"]), "sdd", cfg["mask"].numpy(), False, True)
    assert rel_err(to_np(c), ref) <= 1e-5


def test_config2_dsd_fp16():
    """All 16 heads (the workgroup map takes its second batch group from head 8 on): the oracle on the
    first 2 and the last 2 heads, a dense fp32 product of the same operands on the GPU for all 16, and
    the per-row error (every output row normalised by its own largest reference value) next to the
    global one, so that a mistake confined to rows of small magnitude cannot hide."""
    import sparse, workloads as wl
    cfg = wl.config2(batch=16)
    L = sparse.SparseLayout(cfg["mask"])
    a, b = cfg["a"].cuda(), cfg["b"].cuda()
    c = sparse.matmul(a, b, "dsd", L)
    assert tuple(c.shape) == (16, 2048, 64)
    heads = [0, 1, 14, 15]
    ref = mo.matmul(to_np(cfg["a"][heads]), to_np(cfg["b"][heads]), "dsd", cfg["mask"].numpy())
    assert rel_err(to_np(c[heads]), ref) <= 2e-3
    dense = torch.matmul(L.to_dense(a).float(), b.float())
    err = (c.float() - dense).abs()
    assert (err.max() / dense.abs().max()).item() <= 2e-3
    per_row = err.amax(-1) / dense.abs().amax(-1).clamp_min(1e-6)
    assert per_row.max().item() <= 2e-3


def test_config4_dds_fp16_both_spellings():
    """All 16 heads: the oracle on the first 2 and the last 2 (the workgroup map takes its second batch
    group from head 8 on), a dense fp32 product on the GPU for all 16, rows and tiles on their own."""
    import sparse, workloads as wl
    cfg = wl.config4(batch=16)
    L = sparse.SparseLayout(cfg["mask"])
    a, w = cfg["a"].cuda(), cfg["b"].cuda()
    c = sparse.matmul(a, w, "dds", L, True, False)                 # dY^T W -> [B, 64, 4096]
    assert tuple(c.shape) == (16, 64, 4096)
    heads = [0, 1, 14, 15]
    ref = mo.matmul(to_np(cfg["a"][heads]), to_np(cfg["b"][heads]), "dds", cfg["mask"].numpy(), True, False)
    assert rel_err(to_np(c[heads]), ref) <= 2e-3
    assert local_err(to_np(c[heads]), ref) <= 2e-3
    c2 = sparse.matmul(w, a, "dsd", L, True, False)                # W^T dY -> [B, 4096, 64]
    assert rel_err(to_np(c2[heads]), np.swapaxes(ref, -1, -2)) <= 2e-3
    assert local_err(to_np(c2[heads]), np.swapaxes(ref, -1, -2)) <= 2e-3
    dense = torch.matmul(a.float().transpose(-1, -2), L.to_dense(w).float())
    for got in (c.float(), c2.float().transpose(-1, -2)):
        err = (got - dense).abs()
        assert (err.max() / dense.abs().max()).item() <= 2e-3
        per_column = err.amax(-2) / dense.abs().amax(-2).clamp_min(1e-6)      # every output column (a token) on its own
        assert per_column.max().item() <= 2e-3


def test_full_size_properties_seq4096():
    """Full benchmark size (16 heads): linearity and agreement of the two spellings of one product."""
    import sparse, workloads as wl
    wk = wl.seq4096()
    L = sparse.SparseLayout(wk["mask"])
    q, k, v, w = (wk[n].cuda() for n in ("q", "k", "v", "w"))
    # SDD is linear in a: sdd(2q, k) == 2 * sdd(q, k); a power-of-two scaling is exact in the fp32
    # accumulator and in the fp16 result except where the result is subnormal (spacing 2^-24)
    s1 = sparse.matmul(q, k, "sdd", L, False, True)
    s2 = sparse.matmul(q * 2, k, "sdd", L, False, True)
    normal = s1.abs() >= 2.0 ** -13
    assert torch.equal(s2[normal], (s1 * 2)[normal])
    assert (s2.float() - 2 * s1.float()).abs().max().item() <= 2.0 ** -23
    # DSD against the dense torch product on the GPU (fp32 reference of the same op)
    p = (w.float().abs() * 10).half()
    o = sparse.matmul(p, v, "dsd", L)
    ref = torch.matmul(L.to_dense(p).float(), v.float())
    assert ((o.float() - ref).abs().max() / ref.abs().max()).item() <= 2e-3
    # DDS (dY^T W) equals the transpose of DSD (W^T dY)
    c1 = sparse.matmul(v, w, "dds", L, True, False)
    c2 = sparse.matmul(w, v, "dsd", L, True, False)
    ref = torch.matmul(v.float().transpose(-1, -2), L.to_dense(w).float())
    assert ((c1.float() - ref).abs().max() / ref.abs().max()).item() <= 2e-3
    assert ((c2.float().transpose(-1, -2) - ref).abs().max() / ref.abs().max()).item() <= 2e-3


def test_same_call_twice_is_bit_identical():
    import sparse, workloads as wl
    cfg = wl.config4(batch=2)
    L = sparse.SparseLayout(cfg["mask"])
    a, w = cfg["a"].cuda(), cfg["b"].cuda()
    assert torch.equal(sparse.matmul(a, w, "dds", L, True, False), sparse.matmul(a, w, "dds", L, True, False))


def test_runs_on_the_current_stream():
    import sparse
    mask = np.asarray(ZOO["known3x3"])
    L = sparse.SparseLayout(torch.as_tensor(mask))
    a = torch.randn(1, 96, 64, device="cuda")
    b = torch.randn(1, 96, 64, device="cuda")
    st = torch.cuda.Stream()
    st.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(st):
        c = sparse.matmul(a, b, "sdd", L, False, True)
    st.synchronize()
    assert rel_err(to_np(c), mo.matmul(to_np(a), to_np(b), "sdd", mask, False, True)) <= 1e-5


def test_python_boundary_rejects_misuse():
    import sparse
    from sparse.kernel import sparse_ops
    L = sparse.SparseLayout(torch.as_tensor(np.asarray(ZOO["known3x3"])))
    a = torch.randn(1, 96, 64, device="cuda")
    with pytest.raises(ValueError):
        sparse_ops.sparse_matmul(a, a, "ssd", L.row_layout, L.col_layout, False, True)
    with pytest.raises(TypeError):
        sparse_ops.sparse_matmul(a, a.half(), "sdd", L.row_layout, L.col_layout, False, True)
    with pytest.raises(TypeError):
        sparse_ops.sparse_matmul(a.double(), a.double(), "sdd", L.row_layout, L.col_layout, False, True)
    with pytest.raises(ValueError):
        sparse_ops.sparse_matmul(a[0], a[0], "sdd", L.row_layout, L.col_layout, False, True)   # no batch dim
    with pytest.raises(sparse.kernel.BsaError):
        bad = torch.randn(1, 64, 64, device="cuda")                                            # wrong M
        sparse_ops.sparse_matmul(bad, a, "sdd", L.row_layout, L.col_layout, False, True)
    with pytest.raises(sparse.kernel.BsaError):
        k48 = torch.randn(1, 96, 48, device="cuda")                                            # K % 32
        sparse_ops.sparse_matmul(k48, k48, "sdd", L.row_layout, L.col_layout, False, True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("mode,ta,tb", [(m, x, y) for m in ("dsd", "dds") for x in (False, True) for y in (False, True)])
def test_sparse_operand_shared_by_the_batch(mode, ta, tb, dtype):
    """A sparse input without batch dimensions (a block-sparse weight) serves every batch entry; its
    gradient is the sum over the batch."""
    import sparse
    mask = np.asarray(ZOO["long_col_70x3"] if mode == "dds" else ZOO["rand16"])
    g = torch.Generator().manual_seed(21)
    sa, sb = operand_shapes(mode, mask, 64, ta, tb, (3,))
    if mode == "dsd":
        sa = sa[1:]
    else:
        sb = sb[1:]
    a = torch.randn(sa, generator=g).to(dtype)
    b = torch.randn(sb, generator=g).to(dtype)
    L = sparse.SparseLayout(torch.as_tensor(mask))
    ad, bd = a.cuda().requires_grad_(True), b.cuda().requires_grad_(True)
    c = sparse.matmul(ad, bd, mode, L, ta, tb)
    full_a = a.expand((3,) + tuple(a.shape)) if mode == "dsd" else a
    full_b = b.expand((3,) + tuple(b.shape)) if mode == "dds" else b
    ref = mo.matmul(to_np(full_a), to_np(full_b), mode, mask, ta, tb)
    assert tuple(c.shape) == ref.shape and rel_err(to_np(c), ref) <= tol_of(dtype)
    dc = torch.randn(c.shape, generator=g).to(dtype)
    c.backward(dc.cuda())
    ga, gb = mo.backward(to_np(full_a), to_np(full_b), to_np(dc), mode, mask, ta, tb)
    if mode == "dsd":
        ga = ga.sum(axis=0)
    else:
        gb = gb.sum(axis=0)
    assert ad.grad.shape == ad.shape and bd.grad.shape == bd.shape
    assert rel_err(to_np(ad.grad), ga) <= 2 * tol_of(dtype) and rel_err(to_np(bd.grad), gb) <= 2 * tol_of(dtype)
