"""DSD over runs of block rows (bsa_run_schedule_build, bsa_matmul_dsd_runs): the same product as
``matmul(a, b, 'dsd', layout)`` (sparse/native/sparse_smm_gpu.cu:106-181, dense meaning: dense0(a) @ b),
walked by workgroups that keep the dense strips of a run of consecutive block rows in LDS.

* the schedule: a restatement of the cutting rule in plain Python gives the same runs, and every pair's
  byte names the strip of its own column and marks the first pair of a row;
* the product: against the oracle for every way a row can straddle the waves of a run (runs of one row
  to all rows, 1 to 12 waves, chunks that begin and end inside rows, rows without blocks), through the
  C ABI; and through ``sparse.matmul``, which must take this path for an eligible table.
"""
import numpy as np
import pytest
import torch

from helpers import mask_zoo, rel_err, to_np, tol_of
from oracle import layout_oracle as lo
from oracle import matmul_oracle as mo

pytestmark = pytest.mark.gpu

RECORD_BYTES = 160


def _attention_mask(n=24, window=3, stride=4):
    i, j = np.indices((n, n))
    return ((j <= i) & ((i - j < window) | (j % stride == 0))).astype(np.int64)


def _masks():
    zoo = dict(mask_zoo())
    picked = [(k, zoo[k]) for k in ("known3x3", "single", "one_cell", "full4", "empty_row_col_6x5", "tall_7x2",
                                    "wide_2x9", "rand16", "long_col_70x3")]
    picked.append(("attention24", _attention_mask()))
    first_rows_empty = _attention_mask(12)
    first_rows_empty[:3] = 0
    first_rows_empty[7] = 0
    picked.append(("attention12_empty_rows", first_rows_empty))
    return picked


def _cut_runs(blocks, offsets, target, max_strips):
    """The cutting rule, restated: a row joins the current run unless the run would then name more than
    max_strips distinct columns, or would overshoot the balanced target (nnz / ceil(nnz / target)) by more
    than stopping short of it undershoots."""
    rows, nnz = len(offsets) - 1, int(offsets[-1])
    if any(offsets[r + 1] - offsets[r] > min(max_strips, 64) for r in range(rows)):
        return None
    n_est = -(-nnz // target) if nnz else 1
    runs, byte = [], np.zeros(nnz, np.uint8)
    row0, cols = 0, []
    for r in range(rows):
        row_cols = [int(c) & 0xFFFF for c in blocks[offsets[r]:offsets[r + 1], 1]]
        fresh = [c for c in row_cols if c not in cols]
        cum = offsets[r] - offsets[row0]
        if r > row0 and (len(cols) + len(fresh) > max_strips or (2 * cum + len(row_cols)) * n_est > 2 * nnz):
            runs.append((row0, r, cols))
            row0, cols, fresh = r, [], row_cols
        cols = cols + fresh
        for j, c in enumerate(row_cols):
            byte[offsets[r] + j] = cols.index(c) | (0x80 if j == 0 else 0)
    runs.append((row0, rows, cols))
    return runs, byte


def _build(L, target, max_strips):
    from sparse import _ops
    rs = _ops.RunSchedule(L.row_layout[0], L.row_layout[1], target, max_strips)
    raw = rs.table.cpu().numpy()
    rows = L.row_layout[1].numel() - 1
    records = raw[:rows * RECORD_BYTES].reshape(rows, RECORD_BYTES)
    return rs, records, raw[rows * RECORD_BYTES:]


@pytest.mark.parametrize("target,max_strips", [(1, 39), (5, 39), (96, 39), (7, 4), (1000, 8)])
@pytest.mark.parametrize("name,mask", _masks())
def test_schedule_is_the_restated_cut(name, mask, target, max_strips):
    import sparse
    L = sparse.SparseLayout(torch.as_tensor(mask))
    blocks, offsets = lo.create_layout(mask, False)
    blocks = blocks.reshape(-1, 2)
    blocks = np.stack([blocks[:, 0], blocks[:, 1] & 0xFFFF], axis=1)
    rs, records, pair_byte = _build(L, target, max_strips)
    want = _cut_runs(blocks, offsets, target, max_strips)
    if want is None:
        assert rs.runs == 0 and rs.strips_total == 0
        return
    runs, byte = want
    assert rs.runs == len(runs)
    assert rs.strips == max(len(c) for *_, c in runs) and rs.strips_total == sum(len(c) for *_, c in runs)
    assert rs.pairs == max(offsets[b] - offsets[a] for a, b, _ in runs)
    for k, (a, b, cols) in enumerate(runs):
        head = records[k, :32].view(np.int32)
        assert list(head[:5]) == [a, b, offsets[a], offsets[b], len(cols)], (k, head)
        got = records[k, 32:].view(np.uint16)
        assert list(got[:len(cols)]) == cols
        assert all(c == (cols[-1] if cols else 0) for c in got[len(cols):])
        assert len(cols) <= max_strips
    assert np.array_equal(pair_byte[:len(byte)], byte)
    # what the walk relies on, stated directly
    for a, b, cols in runs:
        for r in range(a, b):
            for p in range(offsets[r], offsets[r + 1]):
                assert cols[pair_byte[p] & 63] == blocks[p, 1]
                assert bool(pair_byte[p] & 0x80) == (p == offsets[r])


@pytest.fixture
def small_launches(monkeypatch):
    """sparse.matmul keeps the run walk for launches that fill the machine; the tests' are small."""
    from sparse import _ops
    monkeypatch.setattr(_ops, "RUN_WALK_PAIRS_MIN", 1)
    monkeypatch.setattr(_ops, "RUN_WALK_PAIRS", 8)
    monkeypatch.setattr(_ops, "RUN_WALK_MIN_REUSE", 0.0)


def test_a_row_longer_than_the_strips_is_not_eligible(small_launches):
    import sparse
    from sparse import _ops
    mask = dict(mask_zoo())["long_row_5x40"]
    L = sparse.SparseLayout(torch.as_tensor(mask))
    rs, _, _ = _build(L, 96, 39)
    assert rs.runs == 0
    assert _ops._run_schedule(L.row_layout, 2, 1) is None
    g = torch.Generator().manual_seed(3)
    a = torch.randn(2, L.num_blocks, 32, 32, generator=g).half()
    b = torch.randn(2, 32 * 40, 64, generator=g).half()
    out = sparse.matmul(a.cuda(), b.cuda(), "dsd", L)              # falls back to the group walk
    assert rel_err(to_np(out), mo.matmul(to_np(a), to_np(b), "dsd", mask)) <= tol_of(torch.float16)


def _call(L, rs, a, b, waves, shared=False):
    from sparse import kernel as K
    rows, cols = L.row_layout[1].numel() - 1, L.col_layout[1].numel() - 1
    batches = b.shape[0]
    out = torch.full((batches, 32 * rows, b.shape[-1]), float("nan"), dtype=a.dtype, device="cuda")
    rc = K.lib.bsa_matmul_dsd_runs(K.BSA_BF16 if a.dtype == torch.bfloat16 else K.BSA_F16, a.data_ptr(), b.data_ptr(),
                                   out.data_ptr(), L.row_layout[0].data_ptr(), L.row_layout[1].data_ptr(),
                                   rs.table.data_ptr(), rs.runs, rs.strips, rs.pairs, waves, rows, cols, L.num_blocks,
                                   batches, 1 if shared else batches, b.shape[-1], K.current_stream())
    return rc, out


@pytest.mark.parametrize("waves", [1, 3, 8, 12])
@pytest.mark.parametrize("target", [1, 7, 1000])
@pytest.mark.parametrize("name,mask", _masks())
def test_product_against_the_oracle(name, mask, target, waves):
    import sparse
    L = sparse.SparseLayout(torch.as_tensor(mask))
    rs, _, _ = _build(L, target, min(39, 4 * waves))
    from sparse import kernel as K
    g = torch.Generator().manual_seed(100 * waves + target)
    a = torch.randn(3, L.num_blocks, 32, 32, generator=g).half()
    b = torch.randn(3, 32 * mask.shape[1], 64, generator=g).half()
    if rs.runs == 0 or rs.pairs > 64 * waves:
        # a row with more blocks than these waves can fetch strips for, or a run too long for them: the build
        # says so (no runs) and the walk refuses what it cannot hold
        assert rs.runs == 0 or rs.pairs > 64 * waves
        rc, _ = _call(L, rs, a.cuda(), b.cuda(), waves)
        assert rc == K.BSA_ERR_INVALID
        return
    rc, out = _call(L, rs, a.cuda(), b.cuda(), waves)
    assert rc == 0
    assert not torch.isnan(out).any()                   # every row written, the empty ones with zeros
    assert rel_err(to_np(out), mo.matmul(to_np(a), to_np(b), "dsd", mask)) <= tol_of(torch.float16)


@pytest.mark.parametrize("dtype,width,batches,shared", [(torch.bfloat16, 64, 2, False), (torch.float16, 128, 17, False),
                                                        (torch.float16, 192, 9, True), (torch.bfloat16, 128, 1, True)])
def test_product_dtypes_widths_batches(dtype, width, batches, shared):
    import sparse
    mask = _attention_mask(40, 4, 8)
    L = sparse.SparseLayout(torch.as_tensor(mask))
    rs, _, _ = _build(L, 48, 32)
    assert rs.runs > 1 and rs.reuse > 2
    g = torch.Generator().manual_seed(width + batches)
    a = torch.randn((L.num_blocks, 32, 32) if shared else (batches, L.num_blocks, 32, 32), generator=g).to(dtype)
    b = torch.randn(batches, 32 * 40, width, generator=g).to(dtype)
    rc, out = _call(L, rs, a.cuda(), b.cuda(), 8, shared)
    assert rc == 0
    a_full = a.expand(batches, *a.shape) if shared else a
    ref = mo.matmul(to_np(a_full), to_np(b), "dsd", mask)
    assert rel_err(to_np(out), ref) <= (1e-2 if dtype == torch.bfloat16 else tol_of(torch.float16))


def test_matmul_takes_the_run_walk_and_agrees_with_the_group_walk(monkeypatch, small_launches):
    import sparse
    from sparse import _ops, kernel as K
    mask = _attention_mask(64, 4, 8)
    L = sparse.SparseLayout(torch.as_tensor(mask))
    g = torch.Generator().manual_seed(64)
    a = torch.randn(2, 4, L.num_blocks, 32, 32, generator=g).half().cuda()
    b = torch.randn(2, 4, 32 * 64, 64, generator=g).half().cuda()
    calls = []
    real_lib = K.lib

    class Spy:
        def __getattr__(self, name):
            if name == "bsa_matmul_dsd_runs":
                return lambda *args: (calls.append(args), real_lib.bsa_matmul_dsd_runs(*args))[1]
            return getattr(real_lib, name)
    monkeypatch.setattr(_ops._k, "lib", Spy())
    out = sparse.matmul(a, b, "dsd", L)
    assert len(calls) == 1
    monkeypatch.setattr(_ops, "RUN_WALK", False)
    old = sparse.matmul(a, b, "dsd", L)
    assert len(calls) == 1
    assert rel_err(to_np(out), to_np(old)) <= tol_of(torch.float16)
    assert rel_err(to_np(out), mo.matmul(to_np(a), to_np(b), "dsd", mask)) <= tol_of(torch.float16)
    # the other DSD variants and fp32 keep the group walk, and so does a launch too small to fill the machine
    monkeypatch.setattr(_ops, "RUN_WALK", True)
    monkeypatch.setattr(_ops, "RUN_WALK_PAIRS_MIN", 48)
    sparse.matmul(a, b, "dsd", L)
    assert len(calls) == 1
    monkeypatch.setattr(_ops, "RUN_WALK_PAIRS_MIN", 1)
    sparse.matmul(a.float(), b.float(), "dsd", L)
    sparse.matmul(a, b.transpose(-1, -2).contiguous(), "dsd", L, False, True)
    assert len(calls) == 1


def test_gradient_through_the_run_walk(small_launches):
    import sparse
    mask = _attention_mask(16, 3, 4)
    L = sparse.SparseLayout(torch.as_tensor(mask))
    g = torch.Generator().manual_seed(5)
    a = torch.randn(2, L.num_blocks, 32, 32, generator=g).half().cuda().requires_grad_()
    b = torch.randn(2, 32 * 16, 64, generator=g).half().cuda().requires_grad_()
    out = sparse.matmul(a, b, "dsd", L)
    go = torch.randn(out.shape, generator=g).half().cuda()
    out.backward(go)
    da, db = mo.backward_dense(to_np(a), to_np(b), to_np(go), "dsd", mask, False, False)
    assert rel_err(to_np(a.grad), da) <= tol_of(torch.float16)
    assert rel_err(to_np(b.grad), db) <= tol_of(torch.float16)


def test_refusals():
    import sparse
    from sparse import kernel as K
    mask = _attention_mask(16, 3, 4)
    L = sparse.SparseLayout(torch.as_tensor(mask))
    rs, _, _ = _build(L, 24, 16)
    a = torch.zeros(1, L.num_blocks, 32, 32, dtype=torch.float16, device="cuda")
    b = torch.zeros(1, 512, 64, dtype=torch.float16, device="cuda")
    assert _call(L, rs, a, b, 13)[0] == K.BSA_ERR_INVALID                       # waves
    assert "waves" in K.lib.bsa_last_error().decode()
    assert rs.strips > 4
    assert _call(L, rs, a, b, 1)[0] == K.BSA_ERR_INVALID                        # more than 4 strips per wave
    assert "strips" in K.lib.bsa_last_error().decode()
    assert _call(L, rs, a, b[..., :32].contiguous(), 8)[0] == K.BSA_ERR_UNSUPPORTED     # width 32
    rows = L.row_layout[1].numel() - 1
    counts = torch.zeros(4, dtype=torch.int32, device="cuda")
    args = (L.row_layout[0].data_ptr(), L.row_layout[1].data_ptr(), rows, L.num_blocks)
    assert K.lib.bsa_run_schedule_build(*args, 0, 8, rs.table.data_ptr(), rs.table.numel(), counts.data_ptr(),
                                        None) == K.BSA_ERR_INVALID              # target
    assert K.lib.bsa_run_schedule_build(*args, 8, 40, rs.table.data_ptr(), rs.table.numel(), counts.data_ptr(),
                                        None) == K.BSA_ERR_INVALID              # strips beyond LDS
    assert K.lib.bsa_run_schedule_build(*args, 8, 8, rs.table.data_ptr(), 16, counts.data_ptr(),
                                        None) == K.BSA_ERR_INVALID              # buffer too small
    assert K.lib.bsa_run_schedule_bytes(rows, L.num_blocks) == RECORD_BYTES * rows + (L.num_blocks + 3) // 4 * 4


def test_headline_size_takes_the_run_walk():
    """4096 tokens, 16 heads, the mask of the benchmark: the launch fills the machine, so ``sparse.matmul`` must walk
    runs (16 per head: one workgroup per compute unit of a 256-unit GPU), and both walks must agree with the dense
    fp32 product computed on the GPU; the run walk twice gives the same bits."""
    import sparse, workloads as wl
    from sparse import _ops
    wk = wl.seq4096()
    L = sparse.SparseLayout(wk["mask"])
    p, v = (wk["w"].float().abs() * 10).half().cuda(), wk["v"].cuda()
    rs = _ops._run_schedule(L.row_layout, 16, 1)
    assert rs is not None and rs.strips <= 32 and rs.reuse > 4
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    assert rs.runs * 16 <= cus or cus != 256
    ref = torch.matmul(L.to_dense(p).float(), v.float())
    out = sparse.matmul(p, v, "dsd", L)
    assert ((out.float() - ref).abs().max() / ref.abs().max()).item() <= tol_of(torch.float16)
    row_err = (out.float() - ref).abs().amax(dim=-1) / ref.abs().amax(dim=-1).clamp_min(1e-6)
    assert row_err.max().item() <= tol_of(torch.float16)
    assert torch.equal(out, sparse.matmul(p, v, "dsd", L))
    _ops.RUN_WALK = False
    try:
        old = sparse.matmul(p, v, "dsd", L)
    finally:
        _ops.RUN_WALK = True
    assert ((old.float() - out.float()).abs().max() / ref.abs().max()).item() <= tol_of(torch.float16)


@pytest.mark.parametrize("seed", range(40))
def test_random_tables_targets_and_waves(seed):
    """Seeded sweep: masks mixing a local window, strided columns, random blocks and empty rows; any target, strip
    limit and wave count the entry point accepts.  Every case against the oracle."""
    import sparse
    from sparse import kernel as K
    rng = np.random.RandomState(1000 + seed)
    rows, cols = int(rng.randint(1, 40)), int(rng.randint(1, 40))
    i, j = np.indices((rows, cols))
    mask = np.zeros((rows, cols), dtype=np.int64)
    if rng.rand() < 0.7:
        mask |= (np.abs(i - j) < rng.randint(1, 4)).astype(np.int64)
    if rng.rand() < 0.6:
        mask |= (j % int(rng.randint(2, 9)) == 0).astype(np.int64)
    mask |= (rng.rand(rows, cols) < rng.choice([0.0, 0.05, 0.3])).astype(np.int64)
    if rng.rand() < 0.5:
        mask &= (j <= i * cols // rows).astype(np.int64)
    mask[rng.rand(rows) < 0.15] = 0
    waves = int(rng.randint(1, 13))
    max_strips = int(rng.randint(1, min(39, 4 * waves) + 1))
    target = int(rng.choice([1, 3, 8, 20, 64, 200]))
    width = 64 * int(rng.randint(1, 3))
    batches = int(rng.choice([1, 2, 9]))
    L = sparse.SparseLayout(torch.as_tensor(mask))
    rs, _, _ = _build(L, target, max_strips)
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(batches, L.num_blocks, 32, 32, generator=g).half()
    b = torch.randn(batches, 32 * cols, width, generator=g).half()
    rc, out = _call(L, rs, a.cuda(), b.cuda(), waves)
    longest = int(mask.sum(axis=1).max())
    if longest > max_strips or rs.pairs > 64 * waves:
        assert (rs.runs == 0) == (longest > max_strips) and rc == K.BSA_ERR_INVALID
        return
    assert rc == 0, K.lib.bsa_last_error()
    assert not torch.isnan(out).any()
    assert rel_err(to_np(out), mo.matmul(to_np(a), to_np(b), "dsd", mask)) <= tol_of(torch.float16)


def test_run_walk_in_a_hip_graph(small_launches):
    """The run walk keeps no state and allocates nothing at launch: captured into a HIP graph after one eager call
    (the schedule is built then), every replay, with other work between the replays, gives the eager result."""
    import sparse
    mask = _attention_mask(32, 3, 4)
    L = sparse.SparseLayout(torch.as_tensor(mask))
    g = torch.Generator().manual_seed(21)
    a = torch.randn(4, L.num_blocks, 32, 32, generator=g).half().cuda()
    b = torch.randn(4, 32 * 32, 64, generator=g).half().cuda()
    eager = sparse.matmul(a, b, "dsd", L)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            out = sparse.matmul(a, b, "dsd", L)
    for r in range(3):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), r
        eager = sparse.matmul(a, b, "dsd", L)          # eager work between the replays


def test_a_schedule_of_another_table_or_launch_is_left_alone():
    """The walk indexes LDS and the operands with what the schedule's records hold.  A schedule cut from another
    table (same number of rows, other pairs), or a launch that reserves fewer strips than a run keeps, must not
    touch memory: the workgroups leave and the result stays as it was."""
    import sparse
    from sparse import kernel as K
    mask = _attention_mask(24, 3, 4)
    other = _attention_mask(24, 2, 6)
    L, L_other = sparse.SparseLayout(torch.as_tensor(mask)), sparse.SparseLayout(torch.as_tensor(other))
    assert L.num_blocks != L_other.num_blocks
    rs_other, _, _ = _build(L_other, 30, 32)
    rs, _, _ = _build(L, 30, 32)
    g = torch.Generator().manual_seed(9)
    a = torch.randn(2, L.num_blocks, 32, 32, generator=g).half().cuda()
    b = torch.randn(2, 32 * 24, 64, generator=g).half().cuda()
    rc, out = _call(L, rs_other, a, b, 8)
    torch.cuda.synchronize()
    assert rc == 0 and torch.isnan(out).all()
    rows = 24
    out = torch.full((2, 32 * rows, 64), float("nan"), dtype=torch.float16, device="cuda")
    assert rs.strips > 2
    rc = K.lib.bsa_matmul_dsd_runs(K.BSA_F16, a.data_ptr(), b.data_ptr(), out.data_ptr(), L.row_layout[0].data_ptr(),
                                   L.row_layout[1].data_ptr(), rs.table.data_ptr(), rs.runs, 2, rs.pairs, 8, rows, rows,
                                   L.num_blocks, 2, 2, 64, K.current_stream())      # claims 2 strips per run
    torch.cuda.synchronize()
    assert rc == 0
    written = ~torch.isnan(out).any(-1).any(0).reshape(rows, 32).any(-1)              # block rows with a result
    assert not written.all()                                                          # the runs that need more left
    ref = mo.matmul(to_np(a), to_np(b), "dsd", mask).reshape(2, rows, 32, 64)
    got = to_np(out).reshape(2, rows, 32, 64)
    for r in range(rows):
        if written[r]:
            assert rel_err(got[:, r], ref[:, r]) <= tol_of(torch.float16)


def test_a_huge_target_is_one_run():
    import sparse
    from sparse import _ops
    mask = _attention_mask(12, 2, 4)
    L = sparse.SparseLayout(torch.as_tensor(mask))
    rs = _ops.RunSchedule(L.row_layout[0], L.row_layout[1], 2 ** 31 - 1, 39)
    assert rs.runs == 1 and rs.pairs == L.num_blocks
