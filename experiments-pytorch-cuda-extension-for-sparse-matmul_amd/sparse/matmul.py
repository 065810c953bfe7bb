"""``matmul``: autograd wrapper of the block-sparse product.

Same Function and call signature as ``sparse/matmul.py:7-57``.  The backward
mode / transpose algebra restates lines 30-50; the products it asks for include
transposed walks the reference kernels get wrong (``sparse_smm_gpu.cu:134,219,287``),
which this build implements by the dense meaning of the operator.
"""
from typing import Any, Optional, Tuple

import torch

from .kernel import sparse_ops
from .layout import SparseLayout


class SparseMatMul(torch.autograd.Function):
    @staticmethod
    def forward(ctx: Any, a: torch.Tensor, b: torch.Tensor, mode: str, layout: SparseLayout,
                trans_a: bool = False, trans_b: bool = False) -> torch.Tensor:
        ctx.save_for_backward(a, b)
        ctx.mode, ctx.layout = mode, layout
        ctx.trans_a, ctx.trans_b = trans_a, trans_b
        return sparse_ops.sparse_matmul(a, b, mode, layout.row_layout, layout.col_layout,
                                        trans_a, trans_b)

    @staticmethod
    def backward(ctx: Any, dc: torch.Tensor) -> Tuple[Optional[torch.Tensor], ...]:
        a, b = ctx.saved_tensors
        mode, layout = ctx.mode, ctx.layout
        trans_a, trans_b = ctx.trans_a, ctx.trans_b
        dc = dc.contiguous()
        da = db = None

        if ctx.needs_input_grad[0]:
            # d op(a) = dc @ op(b)^T, stored back in a's orientation (matmul.py:30-39)
            if trans_a:
                da_mode, lhs, rhs = mode[1] + mode[2] + mode[0], b, dc
            else:
                da_mode, lhs, rhs = mode[1] + mode[0] + mode[2], dc, b
            da = sparse_ops.sparse_matmul(lhs, rhs, da_mode, layout.row_layout, layout.col_layout,
                                          trans_a and trans_b, trans_a or not trans_b)

        if ctx.needs_input_grad[1]:
            # d op(b) = op(a)^T @ dc, stored back in b's orientation (matmul.py:41-50)
            if trans_b:
                db_mode, lhs, rhs = mode[2] + mode[0] + mode[1], dc, a
            else:
                db_mode, lhs, rhs = mode[2] + mode[1] + mode[0], a, dc
            db = sparse_ops.sparse_matmul(lhs, rhs, db_mode, layout.row_layout, layout.col_layout,
                                          not trans_a or trans_b, trans_a and trans_b)

        # a sparse input given without batch dimensions was shared by the batch: its gradient is the sum
        if da is not None and da.dim() > a.dim():
            da = da.sum(dim=tuple(range(da.dim() - a.dim())))
        if db is not None and db.dim() > b.dim():
            db = db.sum(dim=tuple(range(db.dim() - b.dim())))
        return da, db, None, None, None, None


# Call this, not the class (matmul.py:55-57).
matmul = SparseMatMul.apply
