"""``attention``: fused block-sparse attention with autograd.

The reference has no such call: its users chain ``matmul(q, k, 'sdd', layout, False, True)``, a
softmax and ``matmul(p, v, 'dsd', layout)`` (``sparse/matmul.py:57``).  The forward here is ONE
launch that keeps the scores on the chip.  The backward at head dim 64 is two launches that rebuild
the probabilities and the score gradients in registers from the saved row statistics, one walking
the rows (dq), one the columns (dk, dv); at head dim 128 one launch stores them and accumulates dq,
and the two block-sparse products of the unfused chain that walk the columns finish (dk, dv).
"""
from typing import Any, Optional, Tuple

import torch

from .kernel import sparse_ops
from .layout import SparseLayout


class SparseAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx: Any, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, layout: SparseLayout,
                scale: float = 1.0, causal: bool = False) -> torch.Tensor:
        needs_grad = any(t.requires_grad for t in (q, k, v))
        res = sparse_ops.sparse_attention_forward(q, k, v, layout.row_layout[0], layout.row_layout[1],
                                                  scale, causal, layout.col_layout, return_lse=needs_grad)
        out, lse = res if needs_grad else (res, None)
        ctx.save_for_backward(q, k, v, out, lse)
        ctx.layout, ctx.scale, ctx.causal = layout, scale, causal
        return out

    @staticmethod
    def backward(ctx: Any, dout: torch.Tensor) -> Tuple[Optional[torch.Tensor], ...]:
        q, k, v, out, lse = ctx.saved_tensors
        layout = ctx.layout
        rows, cols = layout.row_layout, layout.col_layout
        mm = sparse_ops.sparse_matmul
        dout = dout.contiguous()
        if q.size(-1) == 64:
            # two launches, nothing stored per block: a walk over the rows for dq, one over the columns for dk and dv
            dq, dk, dv = sparse_ops.sparse_attention_backward(q, k, v, dout, out, lse, rows[0], rows[1], cols[0],
                                                              cols[1], ctx.scale, ctx.causal)
            return dq, dk, dv, None, None, None
        # head dim 128: one launch for the probabilities, the score gradients and dq, then the two products
        # over the columns
        p, ds, dq = sparse_ops.sparse_attention_backward_scores(q, k, v, dout, out, lse, rows[0], rows[1],
                                                                ctx.scale, ctx.causal, cols,
                                                                with_dq=ctx.needs_input_grad[0])
        dk = mm(ds, q, "dsd", rows, cols, True, False) if ctx.needs_input_grad[1] else None
        dv = mm(p, dout, "dsd", rows, cols, True, False) if ctx.needs_input_grad[2] else None
        return dq, dk, dv, None, None, None


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, layout: SparseLayout, scale: float = 1.0,
              causal: bool = False) -> torch.Tensor:
    """``softmax(scale * q @ k^T, over the stored blocks of each row) @ v`` for ``q [..., 32 R, D]``,
    ``k``, ``v [..., 32 C, D]`` and an ``R x C`` block layout.  fp16 / bf16 with ``D`` 64 or 128 take the
    fused kernels; fp32, or another ``D`` (a multiple of 32), is computed as the chain of the three
    differentiable operators it stands for."""
    fused = q.dtype in (torch.float16, torch.bfloat16) and q.size(-1) in (64, 128)
    if fused or not (q.dtype == k.dtype == v.dtype and q.dtype in (torch.float16, torch.bfloat16, torch.float32)):
        return SparseAttention.apply(q, k, v, layout, scale, causal)     # the fused path also owns the argument checks
    from .matmul import matmul
    from .softmax import softmax
    scores = matmul(q, k, "sdd", layout, False, True)
    return matmul(softmax(scores, layout, scale, causal), v, "dsd", layout)
