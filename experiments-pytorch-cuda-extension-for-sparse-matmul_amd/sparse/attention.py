"""``attention``: fused block-sparse attention with autograd.

The reference has no such call: its users chain ``matmul(q, k, 'sdd', layout, False, True)``, a
softmax and ``matmul(p, v, 'dsd', layout)`` (``sparse/matmul.py:57``).  The forward here is ONE
launch that keeps the scores on the chip; the backward recomputes the probabilities and goes
through the same block-sparse products and softmax backward as the unfused chain would.
"""
from typing import Any, Optional, Tuple

import torch

from .kernel import sparse_ops
from .layout import SparseLayout


class SparseAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx: Any, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, layout: SparseLayout,
                scale: float = 1.0, causal: bool = False) -> torch.Tensor:
        out = sparse_ops.sparse_attention_forward(q, k, v, layout.row_layout[0], layout.row_layout[1],
                                                  scale, causal, layout.col_layout)
        ctx.save_for_backward(q, k, v)
        ctx.layout, ctx.scale, ctx.causal = layout, scale, causal
        return out

    @staticmethod
    def backward(ctx: Any, dout: torch.Tensor) -> Tuple[Optional[torch.Tensor], ...]:
        q, k, v = ctx.saved_tensors
        layout, scale = ctx.layout, ctx.scale
        rows, cols = layout.row_layout, layout.col_layout
        mm = sparse_ops.sparse_matmul
        dout = dout.contiguous()
        s = mm(q, k, "sdd", rows, cols, False, True)
        p = sparse_ops.sparse_softmax_forward(s, rows[0], rows[1], scale, ctx.causal, cols)
        dp = mm(dout, v, "sdd", rows, cols, False, True)
        ds = sparse_ops.sparse_softmax_backward(p, dp, rows[0], rows[1], scale, cols)
        dq = mm(ds, k, "dsd", rows, cols, False, False) if ctx.needs_input_grad[0] else None
        dk = mm(ds, q, "dsd", rows, cols, True, False) if ctx.needs_input_grad[1] else None
        dv = mm(p, dout, "dsd", rows, cols, True, False) if ctx.needs_input_grad[2] else None
        return dq, dk, dv, None, None, None


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, layout: SparseLayout, scale: float = 1.0,
              causal: bool = False) -> torch.Tensor:
    """``softmax(scale * q @ k^T, over the stored blocks of each row) @ v`` for fp16 / bf16
    ``q [..., 32 R, D]``, ``k``, ``v [..., 32 C, D]``, ``D`` 64 or 128, and an ``R x C`` block layout."""
    return SparseAttention.apply(q, k, v, layout, scale, causal)
