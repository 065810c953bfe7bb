"""Host logic of the boundary: the Python twin of ``sparse_matmul`` in
``sparse/native/sparse_kernels.cc:7-50`` (layout pick, M/N/K rules, batch
flattening, output allocation, dtype dispatch) plus the argument checks the
reference does not make.  ``sparse_matmul`` keeps the reference's positional
signature (``native/sparse_ops.h:10-14``); the softmax entry points keep those of
``sparse_softmax.cu:208-210,233-236`` with ``scale`` / ``causal`` appended.
"""
import torch

from . import kernel as _k

BLOCK = 32
# tuning of the wavefront schedules: (target pairs per wavefront, wavefronts per workgroup)
# (cap, waves, split long groups, no row slicing, -, longest chunks first)
SCHEDULE_GROUP_WALK = (12, 4, True, -1, 2, True)        # groups of at most GROUP_WALK_LONG pairs (rows of attention masks)
SCHEDULE_GROUP_WALK_LONG = (10, 4, True, -1, 2, True)    # tables with longer groups (columns of causal / strided masks)
GROUP_WALK_LONG = 24
SCHEDULE_SDD = (4, 2)
SCHEDULE_SDD_F32 = (1, 4)              # fp32 SDD reloads both operands per block anyway: one block per wave
SCHEDULE_SOFTMAX = (4, 4)
SOFTMAX_LONGEST_FIRST = True     # long rows are dispatched first: they would otherwise finish on a draining machine
SOFTMAX_WAVES_LONG_ROWS = 8
SCHEDULE_BLOCK64 = (4, 2, False)        # coarse pairs (64x64 blocks = four tiles) per wavefront; never split
# DSD on a block=64 layout: True takes the kernel whose wavefronts own whole 64x64 blocks, False walks the layout's
# 32x32 tiles.  Measured at 4096 tokens, 16 heads, 399 blocks of 64 (bench.py, rows block64_mask_*): 17.9-18.8 us
# against 17.1-18.4 us for the group walk over the tiles and 16.5 us for the run walk over them; a wavefront that
# holds a 64 x 64 fp32 tile needs 227 registers (two waves per SIMD), so the tile walks stay the default.
USE_BLOCK64_KERNEL = False
# DSD over a row table with the dense operand stored [K][N]: runs of consecutive block rows whose dense strips stay
# in LDS (bsa_matmul_dsd_runs), when the table is eligible, a fetched strip serves at least RUN_WALK_MIN_REUSE pairs
# and the launch is large enough to give every compute unit a run of RUN_WALK_PAIRS_MIN pairs.  A run is one
# workgroup with a compute unit to itself; the launch is cut into a whole number of generations of about
# RUN_WALK_PAIRS pairs per run (workgroups a few above a multiple of the compute units would cost a generation of
# their own).  Measured at 4096 tokens (1530 blocks per head), DSD fp16, against the walk of bsa_matmul:
# 10.2 / 10.8 / 16.1 / 24.3 / 29.4 / 42.0 us against 12.3 / 12.9 / 16.9 / 26.1 / 33.5 / 44.8 us at
# 4 / 8 / 16 / 24 / 32 / 48 heads.
RUN_WALK = True
RUN_WALK_WAVES = 8
RUN_WALK_PAIRS = 96
RUN_WALK_PAIRS_MIN = 48
RUN_WALK_STRIPS = 32             # 4 per wave; with 10 waves and up to 39 strips (rows of 33-39 blocks) the walk of
                                 # bsa_matmul is 3-6 % faster at 8192 tokens
RUN_WALK_MIN_REUSE = 2.0
ATTENTION_WAVES_LONG_GROUPS = 8
ATTENTION_SPLIT_ROWS = True       # groups longer than cap * waves are cut into parts across workgroups
SCHEDULE_ATTENTION = (12, 4)           # forward: rows of more than 48 blocks are split across workgroups
SCHEDULE_ATTENTION_BACKWARD = (12, 4)
SCHEDULE_ATTENTION_BACKWARD_COLUMNS = (12, 2)
# block rows of at most this many blocks are handed whole to SOFTMAX_SLICES wavefronts (8 element rows
# each), which keep them in registers and need no exchange; per dtype: forward, backward (the
# backward walk keeps two inputs)
SOFTMAX_SLICE_MAX = {torch.float16: (48, 24), torch.bfloat16: (48, 24), torch.float32: (24, 24)}
SOFTMAX_SLICES = {torch.float16: (4, 4), torch.bfloat16: (4, 4), torch.float32: (4, 8)}      # forward, backward

_DTYPES = {torch.float32: _k.BSA_F32, torch.float16: _k.BSA_F16, torch.bfloat16: _k.BSA_BF16}


class Schedule:
    """Device-resident wavefront schedule of one offset table."""

    def __init__(self, offsets: torch.Tensor, nnz: int, cap: int, waves: int, allow_split: bool = True,
                 slice_max: int = -1, slices: int = 2, longest_first: bool = False):
        groups = offsets.numel() - 1
        capacity = _k.lib.bsa_schedule_capacity(groups, nnz, cap, waves)
        self.table = torch.empty(4 * capacity, dtype=torch.int32, device=offsets.device)
        counts = torch.empty(4, dtype=torch.int32, device=offsets.device)
        with torch.cuda.device(offsets.device):
            _k.check(_k.lib.bsa_schedule_build(offsets.data_ptr(), groups, cap, waves,
                                               int(bool(allow_split)) | (2 if longest_first else 0), slice_max,
                                               slices, self.table.data_ptr(), capacity, counts.data_ptr(),
                                               _k.current_stream()))
        self.workgroups, self.tile_slots, self.split_groups, self.slots = (int(v) for v in counts.tolist())
        if self.workgroups < 0:
            raise _k.BsaError("schedule table too small for this offset table")
        self.groups = groups
        self.waves = waves
        self.cap = cap
        self._workspaces = {}
        self._captured = {}
        self._spares = {}
        self.last_key = None

    def workspace(self, mode: int, batches: int, size_m: int, size_n: int, stream: int):
        """Zeroed scratch for split groups, one per (shape, stream): launches on one stream run in
        order and each leaves the buffer zero again; launches on different streams may overlap."""
        need = _k.lib.bsa_matmul_workspace_bytes(mode, self.tile_slots, self.split_groups, batches, size_m, size_n)
        self.last_key = (mode, batches, size_m, size_n, stream)
        return self._zeroed(self.last_key, need)

    def attention_workspace(self, batches: int, head_dim: int, stream: int):
        """The same for the split rows of the fused attention forward."""
        need = _k.lib.bsa_attention_workspace_bytes(self.tile_slots, self.split_groups, batches, head_dim)
        self.last_key = ("attention", batches, head_dim, stream)
        return self._zeroed(self.last_key, need)

    def attention_backward_workspace(self, columns, batches: int, head_dim: int, stream: int):
        """The same for the backward walks: this schedule walks the rows, ``columns`` (or None) the columns."""
        ct, cg = (columns.tile_slots, columns.split_groups) if columns is not None else (0, 0)
        need = _k.lib.bsa_attention_backward_workspace_bytes(self.tile_slots, self.split_groups, ct, cg, batches,
                                                             head_dim)
        self.last_key = ("attention_backward", id(columns), batches, head_dim, stream)
        return self._zeroed(self.last_key, need)

    MAX_WORKSPACES = 16      # eager ones per schedule; the least recently used one goes first

    def _zeroed(self, key, need):
        """Workspace of ``need`` zero bytes for ``key`` (its last item is the stream).  A buffer must be
        zero before its first launch, and under graph capture nothing can be zeroed (a fill recorded
        there only runs at replay, possibly after another graph has used the buffer): every eager call
        keeps one zeroed spare per shape ready, which a first use under capture takes.

        A buffer handed out under capture is never dropped: the captured graph holds its raw address and
        may be replayed at any time.  An eager one is dropped only after the stream it was used on has
        drained (a launch still in flight parks partial tiles there)."""
        if need == 0:
            return None, 0
        capturing = torch.cuda.is_current_stream_capturing()
        spares = self._spares.setdefault(key[:-1], [])
        ws = self._captured.get(key)
        if ws is not None:                              # the graph that owns it is being extended or re-captured
            if not capturing and not spares:
                spares.append(torch.zeros(need, dtype=torch.uint8, device=self.table.device))
            return ws, need
        ws = self._workspaces.pop(key, None)
        if ws is None:
            if capturing:
                if not spares:
                    raise RuntimeError("this operator and shape has never run outside graph capture: call it once "
                                       "eagerly before capturing (its workspace must be zeroed first)")
                ws = spares.pop()
            else:
                ws = torch.zeros(need, dtype=torch.uint8, device=self.table.device)
        if not capturing and not spares:
            spares.append(torch.zeros(need, dtype=torch.uint8, device=self.table.device))
        if capturing:
            self._captured[key] = ws
            return ws, need
        self._workspaces[key] = ws                      # most recently used last
        while len(self._workspaces) > self.MAX_WORKSPACES:
            old_key = next(iter(self._workspaces))
            self._drain(old_key[-1])
            self._workspaces.pop(old_key)
        return ws, need

    def _drain(self, stream_handle):
        """Waits for the stream a workspace was used on before the workspace is given back to the allocator."""
        torch.cuda.ExternalStream(stream_handle, device=self.table.device).synchronize()

    def discard(self, key):
        """Forget the workspace of ``key``: a launch that failed may have left its counters non-zero."""
        self._workspaces.pop(key, None)
        self._captured.pop(key, None)


class RunSchedule:
    """Runs of consecutive block rows of a row table (bsa_run_schedule_build)."""

    def __init__(self, blocks: torch.Tensor, offsets: torch.Tensor, target_pairs: int, max_strips: int):
        rows, nnz = offsets.numel() - 1, blocks.numel() // 2
        need = _k.lib.bsa_run_schedule_bytes(rows, nnz)
        self.table = torch.empty(need, dtype=torch.uint8, device=offsets.device)
        counts = torch.empty(4, dtype=torch.int32, device=offsets.device)
        with torch.cuda.device(offsets.device):
            _k.check(_k.lib.bsa_run_schedule_build(blocks.data_ptr(), offsets.data_ptr(), rows, nnz, target_pairs,
                                                   max_strips, self.table.data_ptr(), need, counts.data_ptr(),
                                                   _k.current_stream()))
        self.runs, self.strips, self.strips_total, self.pairs = (int(v) for v in counts.tolist())
        self.reuse = nnz / self.strips_total if self.strips_total else 0.0


def _run_schedule(layout, batches, strips_n):
    """Run schedule of a row table for a launch of ``batches`` x ``strips_n`` (64-column strips of the result)
    entries, or None when the table is not eligible, the launch is too small to fill the machine with runs, or
    its rows share too few columns for resident strips to pay."""
    blocks, offsets = layout
    nnz = blocks.numel() // 2
    entries = batches * strips_n
    cus = torch.cuda.get_device_properties(offsets.device).multi_processor_count
    if nnz * entries < cus * RUN_WALK_PAIRS_MIN:
        return None
    generations = max(1, round(nnz * entries / (cus * RUN_WALK_PAIRS)))
    runs_wanted = max(1, cus * generations // entries)
    cache = getattr(offsets, "_bsa_runs", None)
    if cache is None:
        cache = {}
        offsets._bsa_runs = cache
    if runs_wanted not in cache:
        if torch.cuda.is_current_stream_capturing():
            return None                     # building synchronises: the first call for a shape runs eagerly
        target = max(RUN_WALK_PAIRS_MIN, -(-nnz // runs_wanted))
        for _ in range(4):                  # a cut forced by the strips can leave one run too many: aim higher
            rs = RunSchedule(blocks, offsets, target, RUN_WALK_STRIPS)
            if rs.runs <= runs_wanted:
                break
            target = -(-target * 11 // 10)
        cache[runs_wanted] = rs
    rs = cache[runs_wanted]
    if rs.runs == 0 or rs.reuse < RUN_WALK_MIN_REUSE:
        return None
    rs.waves = RUN_WALK_WAVES
    return rs if rs.strips <= 4 * rs.waves and rs.pairs <= 64 * rs.waves else None


def _launch(sched, status):
    """Raise on a failed C-ABI call; the workspace the call was given is dropped first, because a launch
    that failed midway may have left its counters non-zero and every later call would sum stale parts."""
    if status != 0 and sched is not None and sched.last_key is not None:
        sched.discard(sched.last_key)
    _k.check(status)


def schedule_for(layout, kind):
    """Schedule of a ``(blocks, offset_table)`` tuple, built on first use and kept
    on the offset tensor (the reference's boundary passes only the two tensors)."""
    blocks, offsets = layout
    cache = getattr(offsets, "_bsa_schedules", None)
    if cache is None:
        cache = {}
        offsets._bsa_schedules = cache
    if kind not in cache:
        cache[kind] = Schedule(offsets, blocks.numel() // 2, *kind)
    return cache[kind]


def _longest_group(offsets) -> int:
    """Pairs in the longest group of a table; measured once and kept on the offsets tensor."""
    longest = getattr(offsets, "_bsa_longest", None)
    if longest is None:
        longest = int((offsets[1:] - offsets[:-1]).max().item()) if offsets.numel() > 1 else 0
        offsets._bsa_longest = longest
    return longest


def _group_walk_schedule(layout):
    kind = SCHEDULE_GROUP_WALK_LONG if _longest_group(layout[1]) > GROUP_WALK_LONG else SCHEDULE_GROUP_WALK
    return schedule_for(layout, kind)


def _attention_schedule(layout, kind, split=False):
    """Schedule of a fused attention walk.  With ``split`` (what every caller passes while
    ``ATTENTION_SPLIT_ROWS`` is set) a group longer than the workgroup's share is cut into parts that
    meet in a workspace; without it such a table gets the most waves a workgroup holds instead."""
    cap, waves = kind
    if split:
        return schedule_for(layout, (cap, waves, True))
    if _longest_group(layout[1]) > cap * waves:
        waves = ATTENTION_WAVES_LONG_GROUPS
    return schedule_for(layout, (cap, waves, False))


def _softmax_schedule(layout, dtype, backward):
    cap, waves = SCHEDULE_SOFTMAX
    which = 1 if backward else 0
    slice_max, slices = SOFTMAX_SLICE_MAX[dtype][which], SOFTMAX_SLICES[dtype][which]
    if _longest_group(layout[1]) > slice_max:
        # a row too long for the register-resident walk is streamed by the waves of ONE workgroup (a row
        # cannot be split across workgroups): as many waves as a workgroup holds keep its chunks short
        waves = SOFTMAX_WAVES_LONG_ROWS
    waves = max(waves, slices)          # the slices of a row share a workgroup
    return schedule_for(layout, (cap, waves, False, slice_max, slices, SOFTMAX_LONGEST_FIRST))


def _check_layout(layout, name):
    blocks, offsets = layout
    for t, what in ((blocks, "blocks"), (offsets, "offset_table")):
        if not (isinstance(t, torch.Tensor) and t.dtype == torch.int32 and t.is_cuda and t.dim() == 1
                and t.is_contiguous()):
            raise ValueError(f"{name}.{what} must be a contiguous 1-D int32 tensor on the GPU")
    if blocks.numel() % 2 or offsets.numel() < 2:
        raise ValueError(f"{name} is malformed")


def sparse_matmul(a, b, mode, row_layout, col_layout, trans_a=False, trans_b=False):
    """``c = op(a) @ op(b)`` with one of a, b, c block-sparse (sparse_kernels.cc:7-50)."""
    if mode not in _k.MODES:
        raise ValueError(f"mode must be one of 'sdd', 'dsd', 'dds', got {mode!r}")
    if a.dtype != b.dtype or a.dtype not in _DTYPES:
        raise TypeError(f"operands must both be float32, float16 or bfloat16, got {a.dtype} and {b.dtype}")
    if not (a.is_cuda and b.is_cuda) or a.device != b.device:
        raise ValueError("operands must live on the same GPU")
    _check_layout(row_layout, "row_layout")
    _check_layout(col_layout, "col_layout")
    trans_a, trans_b = bool(trans_a), bool(trans_b)

    # sparse_kernels.cc:12 : which table the walk uses
    use_row = mode == "sdd" or (mode == "dsd" and not trans_a) or (mode == "dds" and trans_b)
    layout = row_layout if use_row else col_layout
    if layout[0].device != a.device:
        raise ValueError("layout tables and operands must live on the same GPU")
    num_blocks = layout[0].numel() // 2
    mask_rows, mask_cols = row_layout[1].numel() - 1, col_layout[1].numel() - 1
    sparse_width = (layout[1].numel() - 1) * BLOCK                      # :14

    a_dense, b_dense = mode[1] == "d", mode[2] == "d"
    # a sparse INPUT without batch dimensions is shared by every batch entry of the dense operand
    shared = (not a_dense and a.dim() == 3) or (not b_dense and b.dim() == 3)
    if (a_dense and a.dim() < 3) or (b_dense and b.dim() < 3) or (not a_dense and a.dim() < 3) \
            or (not b_dense and b.dim() < 3):
        raise ValueError("operands need at least one batch dimension "
                         "(dense [..., rows, cols], sparse [..., nnz, 32, 32]; a sparse input may "
                         "also be [nnz, 32, 32], shared by the whole batch)")
    for t, dense, name in ((a, a_dense, "a"), (b, b_dense, "b")):
        if not dense and tuple(t.shape[-3:]) != (num_blocks, BLOCK, BLOCK):
            raise ValueError(f"sparse operand {name} must be [..., {num_blocks}, 32, 32], got {tuple(t.shape)}")

    # sparse_kernels.cc:17-19
    size_m = a.size(-1 if trans_a else -2) if a_dense else sparse_width
    size_n = b.size(-2 if trans_b else -1) if b_dense else sparse_width
    size_k = b.size(-1 if trans_b else -2) if b_dense else a.size(-2 if trans_a else -1)
    if a_dense and b_dense and a.size(-2 if trans_a else -1) != size_k:
        raise ValueError("inner dimensions of op(a) and op(b) differ")

    batch_a = tuple(a.shape[:-2] if a_dense else a.shape[:-3])
    batch_b = tuple(b.shape[:-2] if b_dense else b.shape[:-3])
    if shared:
        batch_a = batch_b = batch_a if a_dense else batch_b
    if batch_a != batch_b:
        raise ValueError(f"batch dimensions differ: {batch_a} vs {batch_b} (only a sparse input without "
                         f"batch dimensions is broadcast)")
    batches = 1
    for s in batch_a:
        batches *= s
    if batches < 1:
        raise ValueError("empty batch")

    # :22-37 : flatten the batch, allocate the result
    a = a.contiguous()
    b = b.contiguous()
    if mode[0] == "d":
        shape = batch_a + (size_m, size_n)
    else:
        shape = batch_a + (num_blocks, BLOCK, BLOCK)
    c = torch.empty(shape, dtype=a.dtype, device=a.device)

    coarse = getattr(row_layout[1], "_bsa_coarse", None)
    if (USE_BLOCK64_KERNEL and coarse is not None and mode == "dsd" and not trans_a and not trans_b
            and a.dtype != torch.float32 and size_n % 64 == 0 and num_blocks > 0):
        (cblocks, coffsets), crows, ccols = coarse
        sched = schedule_for((cblocks, coffsets), SCHEDULE_BLOCK64)
        with torch.cuda.device(a.device):
            _k.check(_k.lib.bsa_matmul_dsd_block64(
                _DTYPES[a.dtype], a.data_ptr(), b.data_ptr(), c.data_ptr(), cblocks.data_ptr(), coffsets.data_ptr(),
                sched.table.data_ptr(), sched.workgroups, sched.waves, crows, ccols, cblocks.numel() // 2, batches,
                1 if shared else batches, size_n, _k.current_stream()))
        return c

    if (RUN_WALK and mode == "dsd" and not trans_a and not trans_b and a.dtype != torch.float32
            and size_n % 64 == 0):
        runs = _run_schedule(layout, batches, size_n // 64)
        if runs is not None:
            with torch.cuda.device(a.device):
                _k.check(_k.lib.bsa_matmul_dsd_runs(
                    _DTYPES[a.dtype], a.data_ptr(), b.data_ptr(), c.data_ptr(), layout[0].data_ptr(),
                    layout[1].data_ptr(), runs.table.data_ptr(), runs.runs, runs.strips, runs.pairs, runs.waves,
                    mask_rows, mask_cols, num_blocks, batches, 1 if shared else batches, size_n, _k.current_stream()))
            return c

    if mode == "sdd":
        sched = schedule_for(layout, SCHEDULE_SDD_F32 if a.dtype == torch.float32 else SCHEDULE_SDD)
    else:
        sched = _group_walk_schedule(layout)
    with torch.cuda.device(a.device):
        stream = _k.current_stream()
        ws, ws_bytes = sched.workspace(_k.MODES[mode], batches, size_m, size_n, stream)
        _launch(sched, _k.lib.bsa_matmul(
            _k.MODES[mode], _DTYPES[a.dtype], a.data_ptr(), b.data_ptr(), c.data_ptr(),
            layout[0].data_ptr(), layout[1].data_ptr(), layout[1].numel() - 1,
            sched.table.data_ptr(), sched.workgroups, sched.waves, sched.tile_slots, sched.split_groups,
            ws.data_ptr() if ws is not None else None, ws_bytes,
            mask_rows, mask_cols, num_blocks, batches, 1 if shared else batches, size_m, size_n, size_k,
            int(trans_a), int(trans_b), stream))
    return c


def _softmax_common(x, row_layout, col_layout, name):
    if x.dtype not in _DTYPES:
        raise TypeError(f"{name} must be float32, float16 or bfloat16, got {x.dtype}")
    if not x.is_cuda:
        raise ValueError(f"{name} must live on the GPU")
    _check_layout(row_layout, "row_layout")
    num_blocks = row_layout[0].numel() // 2
    if x.dim() < 4 or tuple(x.shape[-3:]) != (num_blocks, BLOCK, BLOCK):
        raise ValueError(f"{name} must be [..., {num_blocks}, 32, 32] with at least one batch "
                         f"dimension, got {tuple(x.shape)}")
    mask_rows = row_layout[1].numel() - 1
    mask_cols = col_layout[1].numel() - 1 if col_layout is not None else 65535
    batches = x.numel() // max(num_blocks * BLOCK * BLOCK, 1) if num_blocks else 1
    return num_blocks, mask_rows, mask_cols, max(batches, 1)


def sparse_softmax_forward(x, row_blocks, row_table, scale=1.0, causal=False, col_layout=None):
    """``y = softmax(scale * x)`` over the stored blocks of each row (sparse_softmax.cu:208-231)."""
    row_layout = (row_blocks, row_table)
    nnz, mask_rows, mask_cols, batches = _softmax_common(x, row_layout, col_layout, "x")
    x = x.contiguous()
    y = torch.empty_like(x)
    if nnz == 0 or x.numel() == 0:
        return y
    sched = _softmax_schedule(row_layout, x.dtype, False)
    with torch.cuda.device(x.device):
        _k.check(_k.lib.bsa_softmax_forward(
            _DTYPES[x.dtype], x.data_ptr(), y.data_ptr(), row_blocks.data_ptr(), row_table.data_ptr(),
            sched.table.data_ptr(), sched.workgroups, sched.waves, mask_rows, mask_cols, nnz, batches,
            float(scale), int(bool(causal)), _k.current_stream()))
    return y


def sparse_softmax_backward(y, dy, row_blocks, row_table, scale=1.0, col_layout=None):
    """``dx = scale * (dy - sum(dy * y)) * y`` per row (sparse_softmax.cu:233-258)."""
    row_layout = (row_blocks, row_table)
    nnz, mask_rows, mask_cols, batches = _softmax_common(y, row_layout, col_layout, "y")
    if dy.shape != y.shape or dy.dtype != y.dtype or dy.device != y.device:
        raise ValueError("dy must match y in shape, dtype and device")
    y = y.contiguous()
    dy = dy.contiguous()
    dx = torch.empty_like(y)
    if nnz == 0 or y.numel() == 0:
        return dx
    sched = _softmax_schedule(row_layout, y.dtype, True)
    with torch.cuda.device(y.device):
        _k.check(_k.lib.bsa_softmax_backward(
            _DTYPES[y.dtype], y.data_ptr(), dy.data_ptr(), dx.data_ptr(), row_blocks.data_ptr(),
            row_table.data_ptr(), sched.table.data_ptr(), sched.workgroups, sched.waves,
            mask_rows, mask_cols, nnz, batches, float(scale), _k.current_stream()))
    return dx


def _attention_common(q, k, v, row_blocks, row_table, col_layout):
    row_layout = (row_blocks, row_table)
    _check_layout(row_layout, "row_layout")
    for t, name in ((q, "q"), (k, "k"), (v, "v")):
        if t.dtype not in (torch.float16, torch.bfloat16) or t.dtype != q.dtype:
            raise TypeError(f"q, k, v must all be float16 or all bfloat16, got {name}: {t.dtype}")
        if not t.is_cuda or t.device != q.device:
            raise ValueError("q, k, v must live on the same GPU")
        if t.dim() < 3:
            raise ValueError(f"{name} needs at least one batch dimension, got shape {tuple(t.shape)}")
    if row_blocks.device != q.device:
        raise ValueError("layout tables and operands must live on the same GPU")
    if col_layout is None:
        raise ValueError("col_layout is needed for the number of block columns")
    mask_rows, mask_cols = row_table.numel() - 1, col_layout[1].numel() - 1
    head = q.size(-1)
    if q.size(-2) != mask_rows * BLOCK or k.size(-2) != mask_cols * BLOCK or k.shape != v.shape \
            or k.size(-1) != head or q.shape[:-2] != k.shape[:-2]:
        raise ValueError(f"q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)} do not fit a "
                         f"{mask_rows} x {mask_cols} block layout")
    batches = q.numel() // max(q.size(-1) * q.size(-2), 1)
    return row_layout, mask_rows, mask_cols, row_blocks.numel() // 2, head, batches


def sparse_attention_forward(q, k, v, row_blocks, row_table, scale=1.0, causal=False, col_layout=None,
                             return_lse=False):
    """``softmax(scale * q k^T on the stored blocks) v`` in one launch: the chain of
    ``sparse_matmul('sdd', trans_b)``, the softmax and ``sparse_matmul('dsd')`` (sparse/matmul.py:57,
    sparse_softmax.cu:208-231) without the scores in memory.  fp16 / bf16, head dim 64 or 128.
    With ``return_lse`` also the fp32 row statistics the backward pass needs."""
    row_layout, mask_rows, mask_cols, nnz, head, batches = _attention_common(q, k, v, row_blocks, row_table,
                                                                              col_layout)
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    out = torch.empty_like(q)
    lse = torch.empty(q.shape[:-1], dtype=torch.float32, device=q.device) if return_lse else None
    if out.numel() > 0:
        sched = _attention_schedule(row_layout, SCHEDULE_ATTENTION, split=ATTENTION_SPLIT_ROWS)
        with torch.cuda.device(q.device):
            stream = _k.current_stream()
            ws, ws_bytes = sched.attention_workspace(batches, head, stream)
            _launch(sched, _k.lib.bsa_attention_forward(
                _DTYPES[q.dtype], q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                lse.data_ptr() if lse is not None else None,
                row_blocks.data_ptr(), row_table.data_ptr(), sched.table.data_ptr(), sched.workgroups, sched.waves,
                sched.tile_slots, sched.split_groups, ws.data_ptr() if ws is not None else None, ws_bytes,
                mask_rows, mask_cols, nnz, batches, head, float(scale), int(bool(causal)), stream))
    return (out, lse) if return_lse else out


def sparse_attention_backward_scores(q, k, v, dout, out, lse, row_blocks, row_table, scale=1.0, causal=False,
                                     col_layout=None, with_dq=True):
    """Probabilities and score gradients of every stored block, ``[..., nnz, 32, 32]`` each, and (with
    ``with_dq``, else ``None``) the gradient of ``q``, in one launch: what ``sparse_matmul('sdd')``, the
    softmax forward, ``sparse_matmul('sdd')`` on ``dout, v``, the softmax backward
    (sparse_softmax.cu:165-205) and ``sparse_matmul('dsd')`` on ``ds, k`` give with five."""
    row_layout, mask_rows, mask_cols, nnz, head, batches = _attention_common(q, k, v, row_blocks, row_table,
                                                                              col_layout)
    if dout.shape != q.shape or out.shape != q.shape or dout.dtype != q.dtype or out.dtype != q.dtype:
        raise ValueError("dout and out must match q in shape and dtype")
    if lse.dtype != torch.float32 or lse.shape != q.shape[:-1]:
        raise ValueError("lse must be the float32 row statistics of the forward pass")
    q, k, v, dout, out, lse = (t.contiguous() for t in (q, k, v, dout, out, lse))
    shape = q.shape[:-2] + (nnz, BLOCK, BLOCK)
    p = torch.empty(shape, dtype=q.dtype, device=q.device)
    ds = torch.empty(shape, dtype=q.dtype, device=q.device)
    dq = torch.empty_like(q) if with_dq else None
    if q.numel() > 0:
        sched = _attention_schedule(row_layout, SCHEDULE_ATTENTION_BACKWARD, split=ATTENTION_SPLIT_ROWS)
        with torch.cuda.device(q.device):
            stream = _k.current_stream()
            ws, ws_bytes = sched.attention_backward_workspace(None, batches, head, stream) if with_dq else (None, 0)
            _launch(sched, _k.lib.bsa_attention_backward_scores(
                _DTYPES[q.dtype], q.data_ptr(), k.data_ptr(), v.data_ptr(), dout.data_ptr(), out.data_ptr(),
                lse.data_ptr(), p.data_ptr(), ds.data_ptr(), dq.data_ptr() if with_dq else None,
                row_blocks.data_ptr(), row_table.data_ptr(),
                sched.table.data_ptr(), sched.workgroups, sched.waves, sched.tile_slots, sched.split_groups,
                ws.data_ptr() if ws is not None else None, ws_bytes, mask_rows, mask_cols, nnz, batches, head,
                float(scale), int(bool(causal)), stream))
    return p, ds, dq


def sparse_attention_backward(q, k, v, dout, out, lse, row_blocks, row_table, col_blocks, col_table, scale=1.0,
                              causal=False):
    """``(dq, dk, dv)`` of the fused attention in two launches (a walk over the rows, one over the
    columns), the probabilities and score gradients rebuilt in registers in both instead of stored:
    the seven launches of the unfused backward chain (sparse/matmul.py:27-52, sparse_softmax.cu:165-205)
    without a block stack in memory.  fp16 / bf16, head dim 64."""
    col_layout = (col_blocks, col_table)
    _check_layout(col_layout, "col_layout")
    row_layout, mask_rows, mask_cols, nnz, head, batches = _attention_common(q, k, v, row_blocks, row_table,
                                                                              col_layout)
    if head != 64:
        raise ValueError(f"the two-launch backward is built for head dim 64, got {head}")
    if dout.shape != q.shape or out.shape != q.shape or dout.dtype != q.dtype or out.dtype != q.dtype:
        raise ValueError("dout and out must match q in shape and dtype")
    if lse.dtype != torch.float32 or lse.shape != q.shape[:-1]:
        raise ValueError("lse must be the float32 row statistics of the forward pass")
    q, k, v, dout, out, lse = (t.contiguous() for t in (q, k, v, dout, out, lse))
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    if q.numel() > 0:
        delta = torch.empty_like(lse)
        rs = _attention_schedule(row_layout, SCHEDULE_ATTENTION_BACKWARD, split=ATTENTION_SPLIT_ROWS)
        cs = _attention_schedule(col_layout, SCHEDULE_ATTENTION_BACKWARD_COLUMNS, split=ATTENTION_SPLIT_ROWS)
        with torch.cuda.device(q.device):
            stream = _k.current_stream()
            ws, ws_bytes = rs.attention_backward_workspace(cs, batches, head, stream)
            _launch(rs, _k.lib.bsa_attention_backward(
                _DTYPES[q.dtype], q.data_ptr(), k.data_ptr(), v.data_ptr(), dout.data_ptr(), out.data_ptr(),
                lse.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), delta.data_ptr(),
                row_blocks.data_ptr(), row_table.data_ptr(), rs.table.data_ptr(), rs.workgroups, rs.waves,
                rs.tile_slots, rs.split_groups,
                col_blocks.data_ptr(), col_table.data_ptr(), cs.table.data_ptr(), cs.workgroups, cs.waves,
                cs.tile_slots, cs.split_groups, ws.data_ptr() if ws is not None else None, ws_bytes,
                mask_rows, mask_cols, nnz, batches, head, float(scale), int(bool(causal)), stream))
    return dq, dk, dv
