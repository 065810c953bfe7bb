"""``SparseLayout``: block mask -> block-index tables, dense <-> block-stack.

Same class, attributes and methods as ``sparse/layout.py:5-57`` of the
reference.  What changed underneath: the two tables are built by one device
kernel from the uploaded mask (``bsa_layout_build``) instead of CPU torch ops
and four host-to-device copies; ``to_sparse`` / ``to_dense`` of fp16 / fp32 tensors
on the GPU are one copy kernel each (``bsa_to_sparse`` / ``bsa_to_dense``) instead
of Python loops over the blocks, differentiable, and ``to_dense`` fills absent
blocks with zeros (the reference leaves them uninitialised); other tensors (host
memory, other dtypes) take a torch gather; a bool mask means the same as the 0/1
integer mask.

``block=64`` (not in the reference, whose kernels are 32x32x32 only) accepts a mask of
64x64 blocks: the tables and the block stack ``[..., 4 * kept, 32, 32]`` are those of the
mask with each cell repeated twice along both axes, and every operator can run on them as
on any 32x32 layout.  The layout also keeps the row table of the coarse mask
(``coarse_row_layout``, attached to the row offsets so that it travels with the tables
through ``sparse_ops.sparse_matmul``): the untransposed fp16 / bf16 DSD product takes it to
``bsa_matmul_dsd_block64``, whose wavefronts own whole 64x64 blocks.
"""
from typing import Tuple

import torch

from . import kernel as _k

BLOCK = 32
_COPY_DTYPES = {torch.float32: _k.BSA_F32, torch.float16: _k.BSA_F16, torch.bfloat16: _k.BSA_BF16}


class _BlockCopy(torch.autograd.Function):
    """to_sparse (gather = True) / to_dense through the copy kernels; each is the other's gradient."""

    @staticmethod
    def forward(ctx, x, layout, gather):
        ctx.layout, ctx.gather = layout, gather
        return layout._copy_blocks(x, gather)

    @staticmethod
    def backward(ctx, grad):
        return ctx.layout._copy_blocks(grad, not ctx.gather), None, None



class SparseLayout:
    def __init__(self, pattern: torch.Tensor, device=None, block: int = BLOCK):
        if block not in (BLOCK, 2 * BLOCK):
            raise ValueError(f"block must be 32 or 64, got {block}")
        if pattern.dim() != 2:
            raise ValueError("pattern must be a 2-D block mask")
        per_side = block // BLOCK                       # 32x32 tiles along one side of a block
        rows, cols = pattern.size(0) * per_side, pattern.size(1) * per_side
        if not (1 <= rows <= 32767 and 1 <= cols <= 65535):
            raise ValueError("pattern must span [1, 32767] x [1, 65535] tiles of 32x32")
        if device is None:
            device = pattern.device if pattern.is_cuda else torch.device("cuda", torch.cuda.current_device())
        self.pattern = pattern
        self.block = block
        self.tile_shape = (rows, cols)                  # the mask the tables describe, in 32x32 tiles
        self.device = torch.device(device)

        mask = (pattern != 0).to(device=self.device, dtype=torch.uint8)
        if per_side > 1:
            mask = mask.repeat_interleave(per_side, 0).repeat_interleave(per_side, 1)
        mask = mask.contiguous()
        cells = rows * cols
        row_blocks = torch.empty(2 * cells, dtype=torch.int32, device=self.device)
        col_blocks = torch.empty(2 * cells, dtype=torch.int32, device=self.device)
        row_offsets = torch.empty(rows + 1, dtype=torch.int32, device=self.device)
        col_offsets = torch.empty(cols + 1, dtype=torch.int32, device=self.device)
        nnz_dev = torch.empty(1, dtype=torch.int32, device=self.device)
        workspace = torch.empty(_k.lib.bsa_layout_workspace_bytes(rows, cols), dtype=torch.uint8,
                                device=self.device)
        with torch.cuda.device(self.device):
            _k.check(_k.lib.bsa_layout_build(
                mask.data_ptr(), rows, cols, row_blocks.data_ptr(), row_offsets.data_ptr(),
                col_blocks.data_ptr(), col_offsets.data_ptr(), nnz_dev.data_ptr(),
                workspace.data_ptr(), _k.current_stream()))
        nnz = int(nnz_dev.item())
        self.num_blocks = nnz                           # stored 32x32 tiles: the length of a block stack
        self._mask = mask
        self._ordinals = workspace          # int32[rows * cols]: block index of every stored cell
        # exact-size tensors: the boundary derives nnz from blocks.size(0) / 2 (sparse_kernels.cc:13)
        self.row_layout: Tuple[torch.Tensor, torch.Tensor] = (row_blocks[:2 * nnz].clone(), row_offsets)
        self.col_layout: Tuple[torch.Tensor, torch.Tensor] = (col_blocks[:2 * nnz].clone(), col_offsets)

        self.coarse_row_layout = None
        if per_side > 1:
            # row table of the mask in 64x64 blocks, for the kernel that owns whole blocks
            cmask = (pattern != 0).to(device=self.device, dtype=torch.uint8).contiguous()
            crows, ccols = cmask.shape
            cb = torch.empty(2 * crows * ccols, dtype=torch.int32, device=self.device)
            cb2 = torch.empty_like(cb)
            co = torch.empty(crows + 1, dtype=torch.int32, device=self.device)
            co2 = torch.empty(ccols + 1, dtype=torch.int32, device=self.device)
            cws = torch.empty(_k.lib.bsa_layout_workspace_bytes(crows, ccols), dtype=torch.uint8, device=self.device)
            with torch.cuda.device(self.device):
                _k.check(_k.lib.bsa_layout_build(cmask.data_ptr(), crows, ccols, cb.data_ptr(), co.data_ptr(),
                                                 cb2.data_ptr(), co2.data_ptr(), nnz_dev.data_ptr(), cws.data_ptr(),
                                                 _k.current_stream()))
            self.coarse_row_layout = (cb[:nnz // 2].clone(), co)
            self.row_layout[1]._bsa_coarse = (self.coarse_row_layout, crows, ccols)

        packed = self.row_layout[0].view(-1, 2)[:, 1].long()
        # [nnz, 2] (row, col) in row-major order == torch.nonzero(pattern) (layout.py:8)
        self.sparse_positions = torch.stack((packed >> 16, packed & 0xFFFF), dim=1)
        self._cell_index = (self.sparse_positions[:, 0] * cols + self.sparse_positions[:, 1])

    def _index_on(self, device) -> torch.Tensor:
        if self._cell_index.device != device:
            return self._cell_index.to(device)
        return self._cell_index

    def _on_device_path(self, x: torch.Tensor) -> bool:
        return x.is_cuda and x.device == self.device and x.dtype in _COPY_DTYPES

    def _copy_blocks(self, x: torch.Tensor, gather: bool) -> torch.Tensor:
        rows, cols = self.tile_shape
        x = x.contiguous()
        lead = x.shape[:-2] if gather else x.shape[:-3]
        shape = lead + ((self.num_blocks, BLOCK, BLOCK) if gather else (rows * BLOCK, cols * BLOCK))
        out = torch.empty(shape, dtype=x.dtype, device=x.device)
        batches = 1
        for n in lead:
            batches *= n
        if out.numel() == 0 or batches == 0:
            return out
        with torch.cuda.device(self.device):
            if gather:
                _k.check(_k.lib.bsa_to_sparse(_COPY_DTYPES[x.dtype], x.data_ptr(), out.data_ptr(),
                                              self.row_layout[0].data_ptr(), rows, cols, self.num_blocks, batches,
                                              _k.current_stream()))
            else:
                _k.check(_k.lib.bsa_to_dense(_COPY_DTYPES[x.dtype], x.data_ptr(), out.data_ptr(),
                                             self._mask.data_ptr(), self._ordinals.data_ptr(), rows, cols,
                                             self.num_blocks, batches, _k.current_stream()))
        return out

    def to_sparse(self, x: torch.Tensor) -> torch.Tensor:
        """``[..., R*32, C*32]`` -> ``[..., nnz, 32, 32]`` (layout.py:40-45)."""
        rows, cols = self.tile_shape
        if tuple(x.shape[-2:]) != (rows * BLOCK, cols * BLOCK):
            raise ValueError(f"expected [..., {rows * BLOCK}, {cols * BLOCK}], got {tuple(x.shape)}")
        if self._on_device_path(x):
            return _BlockCopy.apply(x, self, True)
        tiles = x.reshape(x.shape[:-2] + (rows, BLOCK, cols, BLOCK)).transpose(-3, -2)
        tiles = tiles.reshape(x.shape[:-2] + (rows * cols, BLOCK, BLOCK))
        return tiles.index_select(-3, self._index_on(x.device)).contiguous()

    def to_dense(self, x: torch.Tensor) -> torch.Tensor:
        """``[..., nnz, 32, 32]`` -> ``[..., R*32, C*32]``, absent blocks zero (layout.py:47-57)."""
        rows, cols = self.tile_shape
        if tuple(x.shape[-3:]) != (self.num_blocks, BLOCK, BLOCK):
            raise ValueError(f"expected [..., {self.num_blocks}, 32, 32], got {tuple(x.shape)}")
        if self._on_device_path(x):
            return _BlockCopy.apply(x, self, False)
        tiles = x.new_zeros(x.shape[:-3] + (rows * cols, BLOCK, BLOCK))
        tiles.index_copy_(-3, self._index_on(x.device), x)
        tiles = tiles.reshape(x.shape[:-3] + (rows, cols, BLOCK, BLOCK)).transpose(-3, -2)
        return tiles.reshape(x.shape[:-3] + (rows * BLOCK, cols * BLOCK))
