"""GPU: the default build against the library built with the compile-time alternative of a hand-rolled
sequence (csrc/build.py, CHECK_VARIANTS), bit for bit.  ``fences``: the parts of a split group publish their
partial tiles with full agent-scope release / acquire fences around the counter (the sequence the memory model
sanctions for any accesses) instead of atomic accesses and a wait for their acknowledgement.
"""
import os

import numpy as np
import pytest
import torch

from helpers import mask_zoo, operand_shapes

pytestmark = pytest.mark.gpu
ZOO = dict(mask_zoo())


def _variant(name):
    import sparse.kernel as k
    path = os.path.join(os.path.dirname(k.LIBRARY_PATH), f"libbsa_hip_{name}.so")
    if not os.path.exists(path):
        pytest.fail(f"{path} is missing: csrc/build.py builds it beside libbsa_hip.so")
    return k.load_library(path)


def _split_masks():
    rng = np.random.RandomState(130)
    big = (rng.rand(130, 130) < 0.06).astype(np.int64)
    big[:, 7] = 1          # a column and a row of 130 blocks: four parts each
    big[5, :] = 1
    return [("long_col_70x3", ZOO["long_col_70x3"]), ("long_row_5x40", ZOO["long_row_5x40"]), ("rand130", big)]


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("mode,ta,tb", [("dsd", False, False), ("dsd", True, False), ("dds", False, False), ("dds", True, True)])
@pytest.mark.parametrize("name,mask", _split_masks(), ids=[n for n, _ in _split_masks()])
def test_fences_around_the_split_counter_give_the_same_bits(name, mask, mode, ta, tb, dtype, monkeypatch):
    import sparse
    import sparse.kernel as k
    from sparse import _ops
    mask = np.asarray(mask)
    L = sparse.SparseLayout(torch.as_tensor(mask))
    sched = _ops._group_walk_schedule(L.row_layout if (mode == "dsd") != ta else L.col_layout)
    g = torch.Generator().manual_seed(11)
    sa, sb = operand_shapes(mode, mask, 128, ta, tb, (3,))
    a, b = torch.randn(sa, generator=g).to(dtype).cuda(), torch.randn(sb, generator=g).to(dtype).cuda()
    monkeypatch.setattr(_ops, "RUN_WALK", False)           # the walk whose groups are split
    want = sparse.matmul(a, b, mode, L, ta, tb)
    if sched.split_groups == 0:
        pytest.skip("no group of the table this variant walks is long enough to be split")
    monkeypatch.setattr(k, "lib", _variant("fences"))
    got = sparse.matmul(a, b, mode, L, ta, tb)
    again = sparse.matmul(a, b, mode, L, ta, tb)
    assert torch.equal(got, want) and torch.equal(again, want)
