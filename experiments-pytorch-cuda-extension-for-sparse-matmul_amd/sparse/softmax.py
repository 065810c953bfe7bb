"""``softmax``: block-sparse row softmax with autograd.

The reference keeps its softmax kernels unbound (``sparse_softmax.cu:208-258``
has the host functions, nothing exports them); this module is the Python face
they would have had, in the style of ``sparse/matmul.py``: an autograd Function
whose forward and backward each make one call through the boundary.
"""
from typing import Any, Optional, Tuple

import torch

from .kernel import sparse_ops
from .layout import SparseLayout


class SparseSoftmax(torch.autograd.Function):
    @staticmethod
    def forward(ctx: Any, x: torch.Tensor, layout: SparseLayout, scale: float = 1.0,
                causal: bool = False) -> torch.Tensor:
        y = sparse_ops.sparse_softmax_forward(x, layout.row_layout[0], layout.row_layout[1],
                                              scale, causal, layout.col_layout)
        ctx.save_for_backward(y)
        ctx.layout, ctx.scale = layout, scale
        return y

    @staticmethod
    def backward(ctx: Any, dy: torch.Tensor) -> Tuple[Optional[torch.Tensor], ...]:
        (y,) = ctx.saved_tensors
        layout = ctx.layout
        dx = sparse_ops.sparse_softmax_backward(y, dy.contiguous(), layout.row_layout[0],
                                                layout.row_layout[1], ctx.scale, layout.col_layout)
        return dx, None, None, None


def softmax(x: torch.Tensor, layout: SparseLayout, scale: float = 1.0, causal: bool = False) -> torch.Tensor:
    """Row softmax of block-sparse scores ``[..., nnz, 32, 32]`` over the stored blocks of each
    row; ``scale`` multiplies the scores first, ``causal`` hides columns right of the diagonal."""
    return SparseSoftmax.apply(x, layout, scale, causal)
