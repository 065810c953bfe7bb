"""TEST INFRASTRUCTURE ONLY (never imported by the product).

CPU restatement of block-sparse attention, ``softmax(scale * q k^T on the stored blocks) v``, in
float64.  The reference has no fused call; its users chain ``sparse.matmul(q, k, 'sdd', layout,
False, True)`` (sparse/matmul.py:57 -> sparse_smm_gpu.cu:22-95), a row softmax over the stored
blocks (sparse_softmax.cu:113-155) and ``sparse.matmul(p, v, 'dsd', layout)``
(sparse_smm_gpu.cu:106-181).  ``forward`` is the dense meaning of that chain, written
independently of the three stage oracles; tests/test_oracle_attention.py pins it against their
composition, against scipy's softmax on full masks and by invariants (rows of weights sum to one,
shift of the logits, permutation of the keys).
"""
import numpy as np


def forward(q, k, v, pattern, scale: float = 1.0, causal: bool = False) -> np.ndarray:
    """q [..., 32 R, D], k and v [..., 32 C, D], pattern R x C -> [..., 32 R, D] in float64.
    Query rows with nothing visible give zeros."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    mask = np.asarray(pattern) != 0
    visible = np.repeat(np.repeat(mask, 32, axis=0), 32, axis=1)
    if causal:
        rows, cols = np.indices(visible.shape)
        visible = visible & (cols <= rows)
    s = scale * np.einsum("...qd,...kd->...qk", q, k)
    s = np.where(visible, s, -np.inf)
    top = np.max(s, axis=-1, keepdims=True)
    top = np.where(np.isfinite(top), top, 0.0)
    w = np.exp(s - top)                       # exp(-inf) = 0 for hidden keys
    den = w.sum(axis=-1, keepdims=True)
    w = np.divide(w, den, out=np.zeros_like(w), where=den > 0)
    return np.einsum("...qk,...kd->...qd", w, v)
