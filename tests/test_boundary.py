"""CPU: the C-ABI library loads, exports what include/bsa.h declares, and validates on the host."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "bsa.h")


@pytest.fixture(scope="module")
def k():
    import sparse.kernel as kernel
    return kernel


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(bsa_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound(k):
    names = _declared()
    assert names == sorted(k.SIGNATURES), "kernel.SIGNATURES must mirror include/bsa.h"
    lib = ctypes.CDLL(k.LIBRARY_PATH)
    for n in names:
        assert hasattr(lib, n), n
    assert k.lib.bsa_version() >= 100
    assert k.lib.bsa_last_error() is not None


def test_missing_library_fails_loudly(k):
    with pytest.raises(ImportError):
        k.load_library("/nonexistent/libbsa_hip.so")


def test_no_product_file_touches_the_oracle():
    pkg = os.path.join(ROOT, "experiments-pytorch-cuda-extension-for-sparse-matmul_amd")
    for base, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h", ".cpp")):
                assert "oracle" not in open(os.path.join(base, f)).read().lower(), f


P = 0x1000  # any non-null address: validation fails before anything is dereferenced or launched


def _matmul(k, mode=0, dtype=1, a=P, b=P, c=P, blocks=P, offs=P, groups=4, sched=P, wgs=1, waves=4,
            tiles=0, splits=0, ws=None, ws_bytes=0,
            R=4, C=4, nnz=5, batches=1, sparse_batches=None, M=128, N=128, K=64, ta=0, tb=1):
    return k.lib.bsa_matmul(mode, dtype, a, b, c, blocks, offs, groups, sched, wgs, waves, tiles, splits,
                            ws, ws_bytes, R, C, nnz, batches, batches if sparse_batches is None else sparse_batches,
                            M, N, K, ta, tb, None)


@pytest.mark.parametrize("kw,needle", [
    (dict(mode=7), "unknown mode"),
    (dict(dtype=5), "unsupported dtype"),
    (dict(a=None), "null pointer"),
    (dict(sched=None), "schedule is null"),
    (dict(K=48), "multiples of 32"),
    (dict(M=96), "layout spans"),
    (dict(groups=3), "groups"),
    (dict(nnz=17), "does not fit"),
    (dict(batches=0), "batches"),
    (dict(batches=3, sparse_batches=2), "sparse_batches"),
    (dict(batches=3, sparse_batches=1), "sparse_batches"),          # sdd has no sparse input to share
    (dict(waves=9), "waves per workgroup"),
    (dict(wgs=0), "workgroups"),
    (dict(mode=1, ta=0, tb=0, M=128, K=96, N=64), "op(sparse a)"),
    (dict(mode=2, ta=0, tb=0, M=64, K=96, N=128), "op(sparse b)"),
    (dict(R=0), "mask shape"),
    (dict(tiles=3, splits=0), "inconsistent"),
    (dict(mode=1, ta=0, tb=0, M=128, K=128, N=64, tiles=4, splits=2), "workspace"),
    (dict(mode=1, ta=0, tb=0, M=128, K=128, N=64, tiles=4, splits=2, ws=P, ws_bytes=100), "workspace"),
])
def test_matmul_validation(k, kw, needle):
    rc = _matmul(k, **kw)
    assert rc < 0
    assert needle in k.lib.bsa_last_error().decode()


def test_other_entry_points_validate(k):
    assert k.lib.bsa_layout_build(None, 4, 4, P, P, P, P, P, P, None) == -1
    assert k.lib.bsa_layout_build(P, 40000, 4, P, P, P, P, P, P, None) == -1
    assert "32767" in k.lib.bsa_last_error().decode()
    assert k.lib.bsa_schedule_build(P, 4, 0, 4, 1, -1, 2, P, 100, P, None) == -1
    assert k.lib.bsa_schedule_build(P, 4, 4, 4, 1, -1, 2, P, 3, P, None) == -1
    assert "capacity" in k.lib.bsa_last_error().decode()
    assert k.lib.bsa_schedule_build(P, 4, 4, 4, 0, 8, 3, P, 100, P, None) == -1
    assert "slices" in k.lib.bsa_last_error().decode()
    assert k.lib.bsa_schedule_build(P, 4, 4, 4, 0, 8, 8, P, 100, P, None) == -1       # 4 waves cannot hold 8 slices
    assert "whole groups" in k.lib.bsa_last_error().decode()
    assert k.lib.bsa_schedule_build(P, 4, 4, 4, 4, -1, 2, P, 100, P, None) == -1
    assert "flags" in k.lib.bsa_last_error().decode()
    assert k.lib.bsa_softmax_forward(3, P, P, P, P, P, 1, 4, 4, 4, 5, 1, 1.0, 0, None) == -3
    assert k.lib.bsa_softmax_forward(1, P, None, P, P, P, 1, 4, 4, 4, 5, 1, 1.0, 0, None) == -1
    assert k.lib.bsa_softmax_backward(1, P, P, P, P, P, P, 1, 4, 4, 4, 5, 0, 1.0, None) == -1
    assert k.lib.bsa_layout_workspace_bytes(4, 8) == 128
    assert k.lib.bsa_schedule_capacity(4, 5, 4, 8) >= 2 * (4 + 1) + 8 + 4
    # workspace: counters (padded to 256 bytes) + one 8 KB fp32 tile per slot, batch and 64-wide strip
    assert k.lib.bsa_matmul_workspace_bytes(0, 4, 2, 3, 128, 128) == 0
    assert k.lib.bsa_matmul_workspace_bytes(1, 0, 0, 3, 128, 128) == 0
    assert k.lib.bsa_matmul_workspace_bytes(1, 4, 2, 3, 128, 128) == 256 + 4 * 3 * 2 * 8192


def test_attention_entry_points_validate(k):
    """Argument checks of the fused attention calls; every case returns before a launch."""
    fwd = lambda dtype=1, head=64, q=P, rows=4, cols=4, nnz=5, batches=1, wgs=4, waves=4, tiles=0, splits=0, ws=None, \
        ws_bytes=0: k.lib.bsa_attention_forward(
            dtype, q, P, P, P, None, P, P, P, wgs, waves, tiles, splits, ws, ws_bytes, rows, cols, nnz, batches, head,
            1.0, 0, None)
    assert fwd(dtype=0) == -3 and "fp16" in k.lib.bsa_last_error().decode()
    assert fwd(head=32) == -3 and "head_dim" in k.lib.bsa_last_error().decode()
    assert fwd(q=None) == -1
    assert fwd(nnz=17) == -1 and "nnz" in k.lib.bsa_last_error().decode()
    assert fwd(rows=0) == -1 and fwd(batches=0) == -1 and fwd(waves=9) == -1
    # split rows: counters (padded to 256 bytes) + per slot and batch entry 32 x head floats of O^T and 128 of (max, sum)
    assert k.lib.bsa_attention_workspace_bytes(0, 0, 3, 64) == 0
    assert k.lib.bsa_attention_workspace_bytes(5, 2, 3, 64) == 256 + 5 * 3 * (32 * 64 + 128) * 4
    assert k.lib.bsa_attention_workspace_bytes(5, 2, 3, 128) == 256 + 5 * 3 * (32 * 128 + 128) * 4
    assert fwd(tiles=3, splits=0) == -1 and "inconsistent" in k.lib.bsa_last_error().decode()
    assert fwd(tiles=5, splits=2) == -1 and "workspace" in k.lib.bsa_last_error().decode()
    assert fwd(tiles=5, splits=2, ws=P, ws_bytes=100) == -1 and "workspace" in k.lib.bsa_last_error().decode()

    scores = lambda p=P, ds=P, dq=P, head=64, lse=P, tiles=0, splits=0, ws=None, ws_bytes=0: \
        k.lib.bsa_attention_backward_scores(1, P, P, P, P, P, lse, p, ds, dq, P, P, P, 4, 4, tiles, splits, ws, ws_bytes,
                                            4, 4, 5, 1, head, 1.0, 0, None)
    assert scores(ds=None) == -1 and "go together" in k.lib.bsa_last_error().decode()
    assert scores(p=None, ds=None, dq=None) == -1 and "no output" in k.lib.bsa_last_error().decode()
    assert scores(lse=None) == -1
    assert scores(head=96) == -3

    assert scores(tiles=2, splits=0) == -1 and "inconsistent" in k.lib.bsa_last_error().decode()
    assert scores(tiles=4, splits=2) == -1 and "workspace" in k.lib.bsa_last_error().decode()

    full = lambda head=64, dk=P, delta=P, col_sched=P, col_waves=4, rt=0, rs=0, ct=0, cs=0, ws=None, ws_bytes=0: \
        k.lib.bsa_attention_backward(1, P, P, P, P, P, P, P, dk, P, delta, P, P, P, 4, 4, rt, rs, P, P, col_sched, 4,
                                     col_waves, ct, cs, ws, ws_bytes, 4, 4, 5, 1, head, 1.0, 0, None)
    assert full(head=128) == -3 and "head_dim 64" in k.lib.bsa_last_error().decode()
    assert full(dk=None) == -1 and full(delta=None) == -1
    assert full(col_sched=None) == -1 and full(col_waves=0) == -1
    # rows: counters + 32 x head floats per slot; columns: counters + 2 x 32 x head floats per slot (dv, dk)
    wsb = k.lib.bsa_attention_backward_workspace_bytes
    assert wsb(0, 0, 0, 0, 3, 64) == 0
    assert wsb(4, 2, 0, 0, 3, 64) == 256 + 4 * 3 * 32 * 64 * 4
    assert wsb(4, 2, 5, 1, 3, 64) == 256 + 4 * 3 * 32 * 64 * 4 + 256 + 5 * 3 * 64 * 64 * 4
    assert full(rt=1, rs=0) == -1 and full(ct=0, cs=3) == -1
    assert full(ct=5, cs=1) == -1 and "workspace" in k.lib.bsa_last_error().decode()
    assert full(ct=5, cs=1, ws=P, ws_bytes=1000) == -1


def test_layout_block_size_is_checked_before_the_device_is_touched():
    import torch
    import sparse
    with pytest.raises(ValueError, match="32 or 64"):
        sparse.SparseLayout(torch.ones(2, 2, dtype=torch.long), block=48)
    with pytest.raises(ValueError, match="2-D"):
        sparse.SparseLayout(torch.ones(2, dtype=torch.long), block=64)
    with pytest.raises(ValueError, match="tiles"):
        sparse.SparseLayout(torch.ones(16384, 1, dtype=torch.long), block=64)     # 32768 tile rows


def test_workspace_is_never_created_under_graph_capture(monkeypatch):
    """A split-group workspace must be zero before its first launch and nothing can be zeroed while a
    graph is being captured: the first use of a shape under capture is refused, a later one on another
    stream takes the buffer an eager call prepared."""
    import torch
    from sparse import _ops
    sched = object.__new__(_ops.Schedule)
    sched._workspaces, sched._captured, sched._spares = {}, {}, {}
    assert sched._zeroed(("attention", 2, 64, 7), 0) == (None, 0)
    monkeypatch.setattr(torch.cuda, "is_current_stream_capturing", lambda: True)
    with pytest.raises(RuntimeError, match="eagerly"):
        sched._zeroed(("attention", 2, 64, 7), 1024)
    spare = torch.zeros(1024, dtype=torch.uint8)
    sched._spares[("attention", 2, 64)] = [spare]
    ws, need = sched._zeroed(("attention", 2, 64, 7), 1024)
    assert ws is spare and need == 1024 and sched._spares[("attention", 2, 64)] == []
    assert sched._zeroed(("attention", 2, 64, 7), 1024)[0] is spare            # kept for that stream
    with pytest.raises(RuntimeError, match="eagerly"):
        sched._zeroed(("attention", 2, 64, 8), 1024)                           # a third stream: nothing prepared
