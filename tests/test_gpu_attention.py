"""GPU: fused block-sparse attention against the float64 oracle and against the unfused chain."""
import numpy as np
import pytest
import torch

from oracle import attention_oracle as ao
from helpers import mask_zoo, rel_err, to_np

pytestmark = pytest.mark.gpu
ZOO = dict(mask_zoo())
TOL = 2e-3          # fp16 operands, fp32 accumulation, probabilities rounded to fp16 (as in the chain)


def _qkv(mask, batch=(2,), seed=0, std=1.0, head=64):
    g = torch.Generator().manual_seed(seed)
    r, c = np.asarray(mask).shape
    mk = lambda n: (std * torch.randn(*batch, 32 * n, head, generator=g)).half()
    return mk(r), mk(c), mk(c)


def _run(mask, scale, causal, **kw):
    import sparse
    q, k, v = _qkv(mask, **kw)
    L = sparse.SparseLayout(torch.as_tensor(np.asarray(mask)))
    out = sparse.attention(q.cuda(), k.cuda(), v.cuda(), L, scale, causal)
    assert out.dtype == torch.float16 and out.shape == q.shape
    return to_np(out), ao.forward(to_np(q), to_np(k), to_np(v), mask, scale, causal)


@pytest.mark.parametrize("scale,causal", [(0.125, False), (0.125, True), (1.0, False), (1.0, True)])
@pytest.mark.parametrize("name", ["known3x3", "single", "one_cell", "full4", "empty_row_col_6x5",
                                  "wide_2x9", "rand16", "long_row_5x40", "long_col_70x3"])
def test_forward(name, scale, causal):
    out, ref = _run(np.asarray(ZOO[name]), scale, causal)
    assert np.all(np.isfinite(out))
    assert rel_err(out, ref) <= TOL


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("name", ["known3x3", "empty_row_col_6x5", "rand16", "long_row_5x40", "long_col_70x3"])
def test_forward_head_dim_128(name, causal):
    out, ref = _run(np.asarray(ZOO[name]), 0.09, causal, head=128, seed=3)
    assert np.all(np.isfinite(out))
    assert rel_err(out, ref) <= TOL


def test_rows_that_see_nothing_give_zeros():
    mask = np.array([[0, 1], [1, 1], [0, 0]])
    out, ref = _run(mask, 1.0, True)
    assert np.all(out[:, :32] == 0) and np.all(out[:, 64:] == 0)       # block (0, 1) is right of the diagonal
    assert rel_err(out, ref) <= TOL


def test_long_rows_and_multi_dim_batch():
    mask = np.zeros((3, 256), dtype=np.int64)
    mask[0, :] = 1
    mask[1, ::5] = 1
    mask[2, 200:] = 1
    out, ref = _run(mask, 0.125, False, batch=(2, 2), seed=4)
    assert rel_err(out, ref) <= TOL


@pytest.mark.parametrize("dtype,head", [(torch.float16, 64), (torch.bfloat16, 64), (torch.float16, 128)])
@pytest.mark.parametrize("causal", [False, True])
def test_rows_split_across_workgroups(dtype, head, causal):
    """Rows longer than one workgroup's share (cap x waves blocks) are cut into parts that meet in a
    workspace: same result as the oracle and, within rounding, as the unsplit walk; a second launch on
    the same workspace gives the same bits (the counters are left at zero); with the causal mask whole
    parts of a row are hidden (their maximum is -inf) and the row statistics still come out right."""
    import sparse
    from sparse import _ops
    rng = np.random.RandomState(9)
    mask = (rng.rand(6, 200) < 0.03).astype(np.int64)
    mask[1, :] = 1                      # 200 blocks: four parts
    mask[3, 10:140] = 1                 # 130 blocks: three parts
    mask[4, :65] = 1                    # 65 blocks: two parts
    mask[5, 150:] = 1                   # all right of the diagonal under the causal mask
    g = torch.Generator().manual_seed(12)
    mk = lambda n: torch.randn(3, 32 * n, head, generator=g).to(dtype)
    q, k, v = mk(6), mk(200), mk(200)
    L = sparse.SparseLayout(torch.as_tensor(mask))
    rl, cl = L.row_layout, L.col_layout
    sched = _ops._attention_schedule(rl, _ops.SCHEDULE_ATTENTION, split=True)
    assert sched.split_groups >= 3 and sched.tile_slots >= 9
    run = lambda: _ops.sparse_attention_forward(q.cuda(), k.cuda(), v.cuda(), rl[0], rl[1], 0.11, causal, cl, return_lse=True)
    out, lse = run()
    out2, lse2 = run()
    assert torch.equal(out, out2) and torch.equal(lse, lse2)
    tol = TOL if dtype == torch.float16 else 1.6e-2
    ref = ao.forward(to_np(q), to_np(k), to_np(v), mask, 0.11, causal)
    assert rel_err(to_np(out), ref) <= tol
    if causal:
        assert torch.all(out[:, 160:] == 0) and torch.all(torch.isinf(lse[:, 160:]))
    try:
        _ops.ATTENTION_SPLIT_ROWS = False
        whole, lse_whole = run()
    finally:
        _ops.ATTENTION_SPLIT_ROWS = True
    assert rel_err(to_np(out), to_np(whole)) <= tol
    seen = torch.isfinite(lse_whole)
    assert torch.equal(seen, torch.isfinite(lse))
    assert torch.allclose(lse[seen], lse_whole[seen], rtol=0, atol=2e-3)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_backward_groups_split_across_workgroups(dtype, causal):
    """Rows and columns longer than one workgroup's share in the two backward walks: parts add up in a
    workspace.  Gradients against the oracle and against the unsplit walks; two launches in a row give
    the same bits (counters left at zero); the stored-stack row walk (dq with p and ds) splits as well."""
    import sparse
    from sparse import _ops
    rng = np.random.RandomState(21)
    mask = (rng.rand(104, 104) < 0.02).astype(np.int64)
    mask[3, :] = 1                      # a row of 104 blocks
    mask[70, 10:90] = 1                 # a row of ~80
    mask[:, 5] = 1                      # a column of 104
    mask[20:100, 99] = 1                # a column of ~80
    g = torch.Generator().manual_seed(33)
    mk = lambda: (0.5 * torch.randn(2, 32 * 104, 64, generator=g)).to(dtype)
    q, k, v, dout = mk(), mk(), mk(), mk()
    L = sparse.SparseLayout(torch.as_tensor(mask))
    rl, cl = L.row_layout, L.col_layout
    rs = _ops._attention_schedule(rl, _ops.SCHEDULE_ATTENTION_BACKWARD, split=True)
    cs = _ops._attention_schedule(cl, _ops.SCHEDULE_ATTENTION_BACKWARD_COLUMNS, split=True)
    assert rs.split_groups >= 2 and cs.split_groups >= 2
    qd, kd, vd, dd = q.cuda(), k.cuda(), v.cuda(), dout.cuda()
    out, lse = _ops.sparse_attention_forward(qd, kd, vd, rl[0], rl[1], 0.125, causal, cl, return_lse=True)
    run = lambda: _ops.sparse_attention_backward(qd, kd, vd, dd, out, lse, rl[0], rl[1], cl[0], cl[1], 0.125, causal)
    grads = run()
    again = run()
    assert all(torch.equal(a, b) for a, b in zip(grads, again))
    ref = ao.backward(to_np(q), to_np(k), to_np(v), to_np(dout), mask, 0.125, causal)
    tol = 4 * TOL if dtype == torch.float16 else 2e-2    # as in test_two_launch_backward
    for name, got, want in zip(("dq", "dk", "dv"), grads, ref):
        assert rel_err(to_np(got), want) <= tol, name
    p, ds, dq = _ops.sparse_attention_backward_scores(qd, kd, vd, dd, out, lse, rl[0], rl[1], 0.125, causal, cl)
    assert rel_err(to_np(dq), ref[0]) <= tol
    try:
        _ops.ATTENTION_SPLIT_ROWS = False
        whole = run()
    finally:
        _ops.ATTENTION_SPLIT_ROWS = True
    for name, a, b in zip(("dq", "dk", "dv"), grads, whole):
        assert rel_err(to_np(a), to_np(b)) <= tol, name


def test_split_rows_at_head_dim_128():
    """The row walk of the backward pass at head dim 128 (four accumulator tiles parked per part)."""
    import sparse
    from sparse import _ops
    mask = np.zeros((4, 120), dtype=np.int64)
    mask[0, :] = 1
    mask[1, ::7] = 1
    mask[2, 30:110] = 1
    mask[3, 5] = 1
    g = torch.Generator().manual_seed(5)
    mk = lambda n: (0.5 * torch.randn(2, 32 * n, 128, generator=g)).half()
    q, k, v, dout = mk(4), mk(120), mk(120), mk(4)
    L = sparse.SparseLayout(torch.as_tensor(mask))
    rl, cl = L.row_layout, L.col_layout
    assert _ops._attention_schedule(rl, _ops.SCHEDULE_ATTENTION_BACKWARD, split=True).split_groups == 2
    out, lse = _ops.sparse_attention_forward(q.cuda(), k.cuda(), v.cuda(), rl[0], rl[1], 0.09, False, cl, return_lse=True)
    assert rel_err(to_np(out), ao.forward(to_np(q), to_np(k), to_np(v), mask, 0.09, False)) <= TOL
    p, ds, dq = _ops.sparse_attention_backward_scores(q.cuda(), k.cuda(), v.cuda(), dout.cuda(), out, lse, rl[0], rl[1],
                                                      0.09, False, cl)
    ref_dq = ao.backward(to_np(q), to_np(k), to_np(v), to_np(dout), mask, 0.09, False)[0]
    assert rel_err(to_np(dq), ref_dq) <= 4 * TOL


def test_large_logits_stay_finite():
    out, ref = _run(np.asarray(ZOO["known3x3"]), 1.0, False, std=6.0, seed=2)   # logits of +-300
    assert np.all(np.isfinite(out)) and rel_err(out, ref) <= TOL


def test_matches_the_unfused_chain_on_config5():
    import sparse, workloads as wl
    cfg = wl.config5()
    L = sparse.SparseLayout(cfg["mask"])
    q, k, v = (cfg[n].cuda() for n in ("q", "k", "v"))
    fused = sparse.attention(q, k, v, L, cfg["scale"], cfg["causal"])
    s = sparse.matmul(q, k, "sdd", L, False, True)
    p = sparse.softmax(s, L, cfg["scale"], cfg["causal"])
    chain = sparse.matmul(p, v, "dsd", L)
    err = ((fused.float() - chain.float()).abs().max() / chain.float().abs().max()).item()
    assert err <= 2e-3
    b, h = 1, 5
    ref = ao.forward(to_np(cfg["q"][b, h][None]), to_np(cfg["k"][b, h][None]), to_np(cfg["v"][b, h][None]),
                     cfg["mask"].numpy(), cfg["scale"], cfg["causal"])
    assert rel_err(to_np(fused[b, h][None]), ref) <= TOL


@pytest.mark.parametrize("head,causal,name", [(64, True, "rand16"), (64, False, "empty_row_col_6x5"), (128, True, "rand16"),
                                              (128, False, "long_row_5x40"), (64, True, "long_col_70x3")])
def test_gradients_match_the_unfused_chain(head, causal, name):
    """Autograd through sparse.attention (two-launch backward at head dim 64, stored-stack backward at 128)
    against the chain of the three differentiable operators and against float64 autograd of the dense meaning."""
    import sparse
    mask = np.asarray(ZOO[name])
    rows, cols = mask.shape
    L = sparse.SparseLayout(torch.as_tensor(mask))
    q, k, v = (t.cuda().requires_grad_(True) for t in _qkv(mask, seed=7, head=head))
    g = torch.randn(q.shape, generator=torch.Generator().manual_seed(8)).half().cuda()
    sparse.attention(q, k, v, L, 0.125, causal).backward(g)
    got = [t.grad.clone() for t in (q, k, v)]
    for t in (q, k, v):
        t.grad = None
    s = sparse.matmul(q, k, "sdd", L, False, True)
    o = sparse.matmul(sparse.softmax(s, L, 0.125, causal), v, "dsd", L)
    o.backward(g)
    for a, t in zip(got, (q, k, v)):
        assert rel_err(to_np(a), to_np(t.grad)) <= 4e-3
    # and against float64 autograd of the dense meaning (rows that see nothing give zeros, not NaN)
    qd, kd, vd = (t.detach().double().cpu().requires_grad_(True) for t in (q, k, v))
    vis = torch.as_tensor(mask).bool().repeat_interleave(32, 0).repeat_interleave(32, 1)
    if causal:
        vis = vis & torch.ones(32 * rows, 32 * cols).tril().bool()
    sc = (0.125 * qd @ kd.transpose(-1, -2)).masked_fill(~vis, float("-inf"))
    p = torch.softmax(sc, -1)
    p = torch.where(vis.any(-1, keepdim=True), p, torch.zeros_like(p))
    (p @ vd).backward(g.double().cpu())
    for a, t in zip(got, (qd, kd, vd)):
        assert rel_err(to_np(a), t.grad.numpy()) <= 4e-3


def test_argument_checks():
    import sparse
    mask = np.asarray(ZOO["known3x3"])
    L = sparse.SparseLayout(torch.as_tensor(mask))
    q, k, v = (t.cuda() for t in _qkv(mask))
    with pytest.raises(TypeError):
        sparse.attention(q.float(), k, v, L)                  # mixed dtypes
    with pytest.raises(TypeError):
        sparse.attention(q.double(), k.double(), v.double(), L)
    with pytest.raises(ValueError):
        sparse.attention(q[:, :64], k, v, L)
    with pytest.raises((ValueError, RuntimeError), match="32"):
        sparse.attention(q[..., :48].contiguous(), k[..., :48].contiguous(), v[..., :48].contiguous(), L)   # not a multiple of 32


@pytest.mark.parametrize("dtype,head,causal", [(torch.float32, 64, True), (torch.float32, 96, False), (torch.float16, 32, True),
                                               (torch.float16, 96, False)])
def test_other_dtypes_and_head_dims_take_the_chain(dtype, head, causal):
    """fp32, and head dims the fused kernels are not built for, go through SDD -> softmax -> DSD, with gradients."""
    import sparse
    mask = np.asarray(ZOO["rand16"])
    L = sparse.SparseLayout(torch.as_tensor(mask))
    q, k, v = (t.to(dtype).cuda().requires_grad_(True) for t in _qkv(mask, seed=31, head=head))
    out = sparse.attention(q, k, v, L, 0.2, causal)
    assert out.dtype == dtype and out.shape == q.shape
    qn, kn, vn = (to_np(t.detach().float()) for t in (q, k, v))
    tol = 1e-5 if dtype == torch.float32 else 2 * TOL
    assert rel_err(to_np(out.detach().float()), ao.forward(qn, kn, vn, mask, 0.2, causal)) <= tol
    g = torch.randn(q.shape, generator=torch.Generator().manual_seed(32)).to(dtype).cuda()
    out.backward(g)
    for got, want in zip((q.grad, k.grad, v.grad), ao.backward(qn, kn, vn, to_np(g.float()), mask, 0.2, causal)):
        assert rel_err(to_np(got.float()), want) <= 2 * tol


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("name,head", [("known3x3", 64), ("rand16", 64), ("long_row_5x40", 64), ("empty_row_col_6x5", 128)])
def test_row_statistics_and_backward_scores(name, head, causal):
    """lse of the forward kernel, and P / dS / dq of the one-launch backward half, against float64."""
    from sparse.kernel import sparse_ops
    from oracle import layout_oracle as lo
    import sparse
    mask = np.asarray(ZOO[name])
    L = sparse.SparseLayout(torch.as_tensor(mask))
    q, k, v = _qkv(mask, seed=17, head=head)
    dout = torch.randn(q.shape, generator=torch.Generator().manual_seed(18)).half()
    scale = 0.11
    rows, cols = L.row_layout, L.col_layout
    out, lse = sparse_ops.sparse_attention_forward(q.cuda(), k.cuda(), v.cuda(), rows[0], rows[1], scale, causal,
                                                   cols, return_lse=True)
    # float64 reference of the dense meaning
    vis = np.repeat(np.repeat(mask != 0, 32, 0), 32, 1)
    if causal:
        r_, c_ = np.indices(vis.shape)
        vis &= c_ <= r_
    s = scale * np.einsum("bqd,bkd->bqk", to_np(q), to_np(k))
    s = np.where(vis, s, -np.inf)
    with np.errstate(divide="ignore"):
        ref_lse = np.log2(np.sum(np.exp(s - np.where(np.isfinite(s.max(-1, keepdims=True)), s.max(-1, keepdims=True), 0)), -1)) \
                  + np.where(np.isfinite(s.max(-1)), s.max(-1), 0) * np.log2(np.e)
    seen = vis.any(axis=1)
    got = to_np(lse)
    assert np.all(np.isposinf(got[:, ~seen]))
    assert np.max(np.abs(got[:, seen] - ref_lse[:, seen])) <= 2e-3 * max(1.0, np.max(np.abs(ref_lse[:, seen])))
    p, ds, dq = sparse_ops.sparse_attention_backward_scores(q.cuda(), k.cuda(), v.cuda(), dout.cuda(), out, lse,
                                                            rows[0], rows[1], scale, causal, cols)
    pd = np.exp(s - np.where(np.isfinite(s.max(-1, keepdims=True)), s.max(-1, keepdims=True), 0))
    den = pd.sum(-1, keepdims=True)
    pd = np.divide(pd, den, out=np.zeros_like(pd), where=den > 0)
    dp = np.einsum("bqd,bkd->bqk", to_np(dout), to_np(v))
    delta = np.sum(to_np(dout) * (pd @ to_np(v)), -1, keepdims=True)
    dsd = scale * pd * (dp - delta)
    assert rel_err(to_np(p), lo.to_sparse(mask, pd)) <= TOL
    assert rel_err(to_np(ds), lo.to_sparse(mask, dsd)) <= 2 * TOL
    assert rel_err(to_np(dq), dsd @ to_np(k)) <= 2 * TOL          # rows without blocks: zeros
    p2, ds2, none = sparse_ops.sparse_attention_backward_scores(q.cuda(), k.cuda(), v.cuda(), dout.cuda(), out, lse,
                                                                rows[0], rows[1], scale, causal, cols, with_dq=False)
    assert none is None and torch.equal(p2, p) and torch.equal(ds2, ds)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("name", ["known3x3", "rand16", "long_row_5x40", "empty_row_col_6x5", "long_col_70x3", "full4",
                                  "tall_7x2", "wide_2x9", "one_cell"])
def test_two_launch_backward(name, dtype, causal):
    """dq, dk, dv of the row walk + column walk (nothing stored per block) against float64."""
    from sparse.kernel import sparse_ops
    import sparse
    mask = np.asarray(ZOO[name])
    L = sparse.SparseLayout(torch.as_tensor(mask))
    q, k, v = (t.to(dtype) for t in _qkv(mask, seed=23, head=64))
    dout = torch.randn(q.shape, generator=torch.Generator().manual_seed(24)).to(dtype)
    scale = 0.13
    rows, cols = L.row_layout, L.col_layout
    out, lse = sparse_ops.sparse_attention_forward(q.cuda(), k.cuda(), v.cuda(), rows[0], rows[1], scale, causal,
                                                   cols, return_lse=True)
    dq, dk, dv = sparse_ops.sparse_attention_backward(q.cuda(), k.cuda(), v.cuda(), dout.cuda(), out, lse,
                                                      rows[0], rows[1], cols[0], cols[1], scale, causal)
    ref_dq, ref_dk, ref_dv = ao.backward(to_np(q.float()), to_np(k.float()), to_np(v.float()), to_np(dout.float()),
                                         mask, scale, causal)
    tol = 4 * TOL if dtype == torch.float16 else 2e-2
    assert rel_err(to_np(dq.float()), ref_dq) <= tol
    assert rel_err(to_np(dk.float()), ref_dk) <= tol
    assert rel_err(to_np(dv.float()), ref_dv) <= tol
    # columns and rows without blocks get zeros, not stale memory
    assert torch.isfinite(dq.float()).all() and torch.isfinite(dk.float()).all() and torch.isfinite(dv.float()).all()
