"""TEST INFRASTRUCTURE ONLY (never imported by the product).

CPU restatement of block-sparse attention, ``softmax(scale * q k^T on the stored blocks) v``, in
float64.  The reference has no fused call; its users chain ``sparse.matmul(q, k, 'sdd', layout,
False, True)`` (sparse/matmul.py:57 -> sparse_smm_gpu.cu:22-95), a row softmax over the stored
blocks (sparse_softmax.cu:113-155) and ``sparse.matmul(p, v, 'dsd', layout)``
(sparse_smm_gpu.cu:106-181).  ``forward`` is the dense meaning of that chain, written
independently of the three stage oracles; tests/test_oracle_attention.py pins it against their
composition, against scipy's softmax on full masks and by invariants (rows of weights sum to one,
shift of the logits, permutation of the keys).  ``backward`` is matrix calculus on that dense meaning
(what the caller's chain computes through sparse/matmul.py:27-52 three times and
sparse_softmax.cu:165-205); the same test file pins it by central finite differences of ``forward``,
by the chain of the stage oracles' backward functions and by torch autograd on a dense restatement.
"""
import numpy as np


def _weights(q, k, pattern, scale, causal):
    """Softmax weights [..., 32 R, 32 C] over the visible keys of every query; zeros where nothing is visible."""
    mask = np.asarray(pattern) != 0
    visible = np.repeat(np.repeat(mask, 32, axis=0), 32, axis=1)
    if causal:
        rows, cols = np.indices(visible.shape)
        visible = visible & (cols <= rows)
    s = np.where(visible, scale * np.einsum("...qd,...kd->...qk", q, k), -np.inf)
    top = np.max(s, axis=-1, keepdims=True)
    top = np.where(np.isfinite(top), top, 0.0)
    w = np.exp(s - top)                       # exp(-inf) = 0 for hidden keys
    den = w.sum(axis=-1, keepdims=True)
    return np.divide(w, den, out=np.zeros_like(w), where=den > 0)


def forward(q, k, v, pattern, scale: float = 1.0, causal: bool = False) -> np.ndarray:
    """q [..., 32 R, D], k and v [..., 32 C, D], pattern R x C -> [..., 32 R, D] in float64.
    Query rows with nothing visible give zeros."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    return np.einsum("...qk,...kd->...qd", _weights(q, k, pattern, scale, causal), v)


def backward(q, k, v, dout, pattern, scale: float = 1.0, causal: bool = False):
    """Gradients (dq, dk, dv) in float64 of ``sum(forward(q, k, v) * dout)``:
    dv = P^T dO;  dP = dO v^T;  dS = scale * P o (dP - rowsum(P o dP));  dq = dS k;  dk = dS^T q."""
    q, k, v, dout = (np.asarray(t, dtype=np.float64) for t in (q, k, v, dout))
    p = _weights(q, k, pattern, scale, causal)
    dv = np.einsum("...qk,...qd->...kd", p, dout)
    dp = np.einsum("...qd,...kd->...qk", dout, v)
    ds = scale * p * (dp - np.sum(p * dp, axis=-1, keepdims=True))
    return np.einsum("...qk,...kd->...qd", ds, k), np.einsum("...qk,...qd->...kd", ds, q), dv
