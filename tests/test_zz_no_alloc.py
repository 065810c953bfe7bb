"""GPU: bsa_matmul_noalloc (the entry point that allocates nothing) against bsa_matmul, through the C ABI.

Both entry points launch the same kernels, the only difference being where the partial tiles and
counters of split groups live, and parts are summed in part order, so the results must be identical
bit for bit.  Two calls in a row share the library's static scratch buffer, the second on a smaller
input: whatever the first left behind must not leak into it.
"""
import ctypes

import numpy as np
import pytest
import torch

from oracle import matmul_oracle as mo
from helpers import mask_zoo, operand_shapes, rel_err, to_np, tol_of

pytestmark = pytest.mark.gpu

ZOO = dict(mask_zoo())


def _call(entry, mode, a, b, layout, sched, ta, tb, M, N, K, batches, workspace):
    """One call of `entry` ("bsa_matmul" or "bsa_matmul_noalloc") with raw pointers; returns c."""
    from sparse import kernel as k
    rows, cols = layout.row_layout, layout.col_layout
    use_row = (mode == "dsd" and not ta) or (mode == "dds" and tb)
    blocks, offsets = rows if use_row else cols
    c = torch.empty((batches, M, N), dtype=a.dtype, device=a.device)
    dtype = {torch.float32: k.BSA_F32, torch.float16: k.BSA_F16}[a.dtype]
    head = (k.MODES[mode], dtype, a.data_ptr(), b.data_ptr(), c.data_ptr(), blocks.data_ptr(), offsets.data_ptr(),
            offsets.numel() - 1, sched.table.data_ptr(), sched.workgroups, sched.waves, sched.tile_slots,
            sched.split_groups)
    tail = (rows[1].numel() - 1, cols[1].numel() - 1, blocks.numel() // 2, batches, batches, M, N, K, int(ta), int(tb),
            k.current_stream())
    if entry == "bsa_matmul":
        need = k.lib.bsa_matmul_workspace_bytes(k.MODES[mode], sched.tile_slots, sched.split_groups, batches, M, N)
        assert workspace is not None and workspace.numel() >= need
        k.check(k.lib.bsa_matmul(*head, workspace.data_ptr(), ctypes.c_size_t(workspace.numel()), *tail))
    else:
        k.check(k.lib.bsa_matmul_noalloc(*head, *tail))
    return c


def _case(mode, ta, tb, mask, free, batches, dtype, seed, cap_waves):
    import sparse
    from sparse import _ops
    mask = np.asarray(mask)
    g = torch.Generator().manual_seed(seed)
    sa, sb = operand_shapes(mode, mask, free, ta, tb, (batches,))
    a = torch.randn(sa, generator=g).to(dtype).cuda()
    b = torch.randn(sb, generator=g).to(dtype).cuda()
    layout = sparse.SparseLayout(torch.as_tensor(mask))
    use_row = (mode == "dsd" and not ta) or (mode == "dds" and tb)
    table = layout.row_layout if use_row else layout.col_layout
    sched = _ops.Schedule(table[1], table[0].numel() // 2, cap_waves[0], cap_waves[1], True, -1, 2, True)
    R, C = mask.shape
    if mode == "dsd":
        M, K, N = (32 * C, 32 * R, free) if ta else (32 * R, 32 * C, free)
    else:
        M, K, N = (free, 32 * C, 32 * R) if tb else (free, 32 * R, 32 * C)
    ref = mo.matmul(to_np(a), to_np(b), mode, mask, ta, tb)
    return dict(mode=mode, a=a, b=b, layout=layout, sched=sched, ta=ta, tb=tb, M=M, N=N, K=K, batches=batches), ref


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("mode,ta,tb", [("dds", False, False), ("dsd", True, False), ("dsd", False, False)])
def test_noalloc_matches_matmul_on_two_calls_in_a_row(mode, ta, tb, dtype):
    from sparse import kernel as k
    # first call: a column (row) of 70 (40) blocks cut into many parts, three 64-wide strips, 3 batch entries;
    # second call: a smaller input (one strip, one batch entry, fewer parts) on the same scratch buffer
    big_mask = ZOO["long_row_5x40"] if (mode == "dsd" and not ta) else ZOO["long_col_70x3"]
    small_mask = big_mask[:, :17] if (mode == "dsd" and not ta) else big_mask[:23]
    first, ref1 = _case(mode, ta, tb, big_mask, 160, 3, dtype, 1, (2, 2))
    second, ref2 = _case(mode, ta, tb, small_mask, 64, 1, dtype, 2, (3, 2))
    for case in (first, second):
        assert case["sched"].split_groups > 0, "the case must exercise split groups"
    results = []
    for case, ref in ((first, ref1), (second, ref2)):
        s = case["sched"]
        need = k.lib.bsa_matmul_workspace_bytes(k.MODES[mode], s.tile_slots, s.split_groups, case["batches"],
                                                case["M"], case["N"])
        assert 0 < need <= 16 << 20
        ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
        want = _call("bsa_matmul", workspace=ws, **case)
        got = _call("bsa_matmul_noalloc", workspace=None, **case)
        torch.cuda.synchronize()
        results.append((got, want, ref))
    for got, want, ref in results:
        assert torch.equal(got, want)                               # same kernels, same order of the parts
        assert rel_err(to_np(got), ref) <= tol_of(dtype)            # and both are right


def test_noalloc_without_split_groups_and_sdd():
    """Schedules that need no scratch, and SDD (which never does), go through the same entry point."""
    import sparse
    from sparse import kernel as k, _ops
    case, ref = _case("dsd", False, False, ZOO["known3x3"], 64, 2, torch.float16, 3, (10, 4))
    assert case["sched"].split_groups == 0
    got = _call("bsa_matmul_noalloc", workspace=None, **case)
    assert rel_err(to_np(got), ref) <= tol_of(torch.float16)
    # sdd
    mask = np.asarray(ZOO["rand16"])
    g = torch.Generator().manual_seed(4)
    a = torch.randn(2, 512, 64, generator=g).half().cuda()
    b = torch.randn(2, 512, 64, generator=g).half().cuda()
    layout = sparse.SparseLayout(torch.as_tensor(mask))
    rows = layout.row_layout
    sched = _ops.schedule_for(rows, _ops.SCHEDULE_SDD)
    nnz = rows[0].numel() // 2
    c = torch.empty((2, nnz, 32, 32), dtype=torch.float16, device="cuda")
    k.check(k.lib.bsa_matmul_noalloc(k.BSA_SDD, k.BSA_F16, a.data_ptr(), b.data_ptr(), c.data_ptr(), rows[0].data_ptr(),
                                     rows[1].data_ptr(), 16, sched.table.data_ptr(), sched.workgroups, sched.waves,
                                     sched.tile_slots, sched.split_groups, 16, 16, nnz, 2, 2, 512, 512, 64, 0, 1,
                                     k.current_stream()))
    assert rel_err(to_np(c), mo.matmul(to_np(a), to_np(b), "sdd", mask, False, True)) <= tol_of(torch.float16)


def test_noalloc_refuses_more_scratch_than_it_has():
    """A schedule whose split groups need more than the static buffer is refused before any launch."""
    from sparse import kernel as k
    case, _ = _case("dds", False, False, ZOO["long_col_70x3"], 64, 1, torch.float16, 5, (2, 2))
    s = case["sched"]
    batches = 4096                      # the need grows with the batch: far beyond 16 MiB
    need = k.lib.bsa_matmul_workspace_bytes(k.BSA_DDS, s.tile_slots, s.split_groups, batches, case["M"], case["N"])
    assert need > 16 << 20
    rows, cols = case["layout"].row_layout, case["layout"].col_layout
    blocks, offsets = cols
    dummy = case["a"].data_ptr()        # never dereferenced: the call fails validation
    rc = k.lib.bsa_matmul_noalloc(k.BSA_DDS, k.BSA_F16, dummy, case["b"].data_ptr(), dummy, blocks.data_ptr(),
                                  offsets.data_ptr(), offsets.numel() - 1, s.table.data_ptr(), s.workgroups, s.waves,
                                  s.tile_slots, s.split_groups, rows[1].numel() - 1, cols[1].numel() - 1,
                                  blocks.numel() // 2, batches, batches, case["M"], case["N"], case["K"], 0, 0,
                                  k.current_stream())
    assert rc == -3 and b"static buffer" in k.lib.bsa_last_error()


def test_noalloc_allocates_nothing_and_replays_from_a_graph():
    """What the entry point is for.  After one eager call on the device (which looks up the scratch array's
    address), a call with split groups is captured on a side stream and replayed; between the replays an eager
    call of another shape uses, and dirties, the same scratch.  Every replay must give bsa_matmul's bits, and the
    device allocator must hold exactly what it held before."""
    from sparse import kernel as k
    case, ref = _case("dds", False, False, ZOO["long_col_70x3"], 128, 2, torch.float16, 7, (2, 2))
    other, _ = _case("dsd", False, False, ZOO["long_row_5x40"], 64, 3, torch.float16, 8, (3, 2))
    assert case["sched"].split_groups > 0 and other["sched"].split_groups > 0
    s = case["sched"]
    need = k.lib.bsa_matmul_workspace_bytes(k.BSA_DDS, s.tile_slots, s.split_groups, case["batches"], case["M"], case["N"])
    want = _call("bsa_matmul", workspace=torch.zeros(need, dtype=torch.uint8, device="cuda"), **case)
    _call("bsa_matmul_noalloc", workspace=None, **other)          # first call on this device: outside capture
    torch.cuda.synchronize()

    out = torch.empty_like(want)
    head = (k.BSA_DDS, k.BSA_F16, case["a"].data_ptr(), case["b"].data_ptr(), out.data_ptr(),
            case["layout"].col_layout[0].data_ptr(), case["layout"].col_layout[1].data_ptr(),
            case["layout"].col_layout[1].numel() - 1, s.table.data_ptr(), s.workgroups, s.waves, s.tile_slots, s.split_groups)
    tail = (case["layout"].row_layout[1].numel() - 1, case["layout"].col_layout[1].numel() - 1,
            case["layout"].col_layout[0].numel() // 2, case["batches"], case["batches"], case["M"], case["N"], case["K"], 0, 0)
    torch.cuda.synchronize()
    before = (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.mem_get_info()[0])
    k.check(k.lib.bsa_matmul_noalloc(*head, *tail, k.current_stream()))
    torch.cuda.synchronize()
    after = (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.mem_get_info()[0])
    assert after == before, (before, after)
    assert torch.equal(out, want)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        out.fill_(float("nan"))
        with torch.cuda.graph(graph, stream=side):
            k.check(k.lib.bsa_matmul_noalloc(*head, *tail, k.current_stream()))
    for replay in range(3):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), replay
        _call("bsa_matmul_noalloc", workspace=None, **other)      # the same scratch, another shape, in between
        torch.cuda.synchronize()
    assert rel_err(to_np(out), ref) <= tol_of(torch.float16)
