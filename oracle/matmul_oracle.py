"""SDD / DSD / DDS block-sparse matmul: dense semantics in float64 (CPU oracle).

TEST INFRASTRUCTURE ONLY: nothing shipped imports this file.

The meaning of ``matmul(a, b, mode, layout, trans_a, trans_b)`` is the one the
host dispatcher of the reference encodes in its shape rules,
``sparse/native/sparse_kernels.cc:12-37``: mode is three letters
``[out][a][b]``, each ``s`` (block-sparse, stored ``[..., nnz, 32, 32]``) or
``d`` (dense):

``sdd``  ``to_sparse(op(a) @ op(b))``
``dsd``  ``op(dense0(a)) @ op(b)``
``dds``  ``op(a) @ op(dense0(b))``

with ``op(x) = x`` or its transpose over the last two dims and ``dense0`` the
zero-filled ``to_dense``.  Several transposed paths of the reference kernels
index the wrong coordinate (``sparse_smm_gpu.cu:134,219,287``); the dense
meaning above is the contract, not those outputs.

The backward rule restates ``sparse/matmul.py:30-50``.
"""
import numpy as np

from . import layout_oracle as lo


def _t(x):
    return np.swapaxes(x, -1, -2)


def matmul(a, b, mode: str, pattern, trans_a: bool = False, trans_b: bool = False):
    """float64 result of the dense meaning; inputs are used at their stored values."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    if mode not in ("sdd", "dsd", "dds"):
        raise ValueError(mode)
    if mode[1] == "s":
        a = lo.to_dense(pattern, a, 0.0)
    if mode[2] == "s":
        b = lo.to_dense(pattern, b, 0.0)
    c = np.matmul(_t(a) if trans_a else a, _t(b) if trans_b else b)
    if mode[0] == "s":
        c = lo.to_sparse(pattern, c)
    return c


def backward_plan(mode: str, trans_a: bool, trans_b: bool):
    """The two follow-up products of ``SparseMatMul.backward`` (sparse/matmul.py:30-50).

    Returns ``(da_plan, db_plan)``; each plan is ``(lhs, rhs, mode, ta, tb)``
    with ``lhs``/``rhs`` in ``{"a", "b", "dc"}``.
    """
    if trans_a:
        da = ("b", "dc", mode[1] + mode[2] + mode[0])
    else:
        da = ("dc", "b", mode[1] + mode[0] + mode[2])
    da += (trans_a and trans_b, trans_a or not trans_b)
    if trans_b:
        db = ("dc", "a", mode[2] + mode[0] + mode[1])
    else:
        db = ("a", "dc", mode[2] + mode[1] + mode[0])
    db += (not trans_a or trans_b, trans_a and trans_b)
    return da, db


def backward(a, b, dc, mode, pattern, trans_a=False, trans_b=False):
    """Gradients by running the plan through :func:`matmul`."""
    env = {"a": a, "b": b, "dc": dc}
    da_p, db_p = backward_plan(mode, trans_a, trans_b)
    da = matmul(env[da_p[0]], env[da_p[1]], da_p[2], pattern, da_p[3], da_p[4])
    db = matmul(env[db_p[0]], env[db_p[1]], db_p[2], pattern, db_p[3], db_p[4])
    return da, db


def backward_dense(a, b, dc, mode, pattern, trans_a=False, trans_b=False):
    """Gradients from matrix calculus on the dense meaning, independent of
    :func:`backward_plan`: for ``C = op(A) op(B)``, ``d op(A) = dC op(B)^T`` and
    ``d op(B) = op(A)^T dC``, masked to the stored blocks for sparse operands."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    dc = np.asarray(dc, dtype=np.float64)
    ad = lo.to_dense(pattern, a, 0.0) if mode[1] == "s" else a
    bd = lo.to_dense(pattern, b, 0.0) if mode[2] == "s" else b
    dcd = lo.to_dense(pattern, dc, 0.0) if mode[0] == "s" else dc
    opa = _t(ad) if trans_a else ad
    opb = _t(bd) if trans_b else bd
    d_opa = np.matmul(dcd, _t(opb))
    d_opb = np.matmul(_t(opa), dcd)
    da = _t(d_opa) if trans_a else d_opa
    db = _t(d_opb) if trans_b else d_opb
    if mode[1] == "s":
        da = lo.to_sparse(pattern, da)
    if mode[2] == "s":
        db = lo.to_sparse(pattern, db)
    return da, db


def rel_err(out, ref) -> float:
    """max|out - ref| / max|ref| : the parity metric for floating-point results."""
    out = np.asarray(out, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    denom = float(np.max(np.abs(ref))) if ref.size else 0.0
    if ref.size == 0:
        return 0.0
    return float(np.max(np.abs(out - ref))) / (denom if denom > 0 else 1.0)
