"""The reference-side binding of the integration notes ("Option B"): the code block a maintainer of the
reference would paste as sparse/kernel.py is taken out of the document and executed as it stands.

Without a GPU: it loads the library and its ctypes signatures agree with the bindings of this package.
With a GPU: its ``sparse_ops.sparse_matmul`` (the reference's pybind name and positional signature,
sparse/native/sparse_kernels.cc:53-57) gives the oracle's results for sdd / dsd / dds on a mask with a
column long enough to be split across workgroups.
"""
import os
import re

import numpy as np
import pytest
import torch

from helpers import mask_zoo, operand_shapes, rel_err, to_np, tol_of
from oracle import matmul_oracle as mo

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _stub_namespace():
    from sparse import kernel as k
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    section = text[text.index("## Option B"):]
    code = re.search(r"```python\n(.*?)```", section, re.S).group(1)
    assert '"libbsa_hip.so"' in code
    ns = {}
    exec(compile(code.replace('"libbsa_hip.so"', repr(k.LIBRARY_PATH)), "<Option B stub>", "exec"), ns)
    return ns


def test_stub_loads_and_its_signatures_match_the_package():
    from sparse import kernel as k
    ns = _stub_namespace()
    lib = ns["_lib"]
    for name in ("bsa_schedule_build", "bsa_matmul_workspace_bytes", "bsa_matmul"):
        restype, argtypes = k.SIGNATURES[name]
        assert list(getattr(lib, name).argtypes) == argtypes, name
    assert lib.bsa_schedule_capacity.restype is k.SIGNATURES["bsa_schedule_capacity"][0]
    assert lib.bsa_matmul_workspace_bytes.restype is k.SIGNATURES["bsa_matmul_workspace_bytes"][0]
    assert callable(ns["sparse_ops"].sparse_matmul)


@pytest.mark.gpu
@pytest.mark.parametrize("mode,ta,tb", [("sdd", False, True), ("dsd", False, False), ("dsd", True, False),
                                        ("dds", True, False), ("dds", False, True)])
def test_stub_sparse_matmul_against_the_oracle(mode, ta, tb):
    import sparse
    ns = _stub_namespace()
    mask = np.asarray(dict(mask_zoo())["long_col_70x3"])
    layout = sparse.SparseLayout(torch.as_tensor(mask))        # this repository's tables (same format as the reference's)
    g = torch.Generator().manual_seed(11)
    sa, sb = operand_shapes(mode, mask, 64, ta, tb, (2,))
    a = torch.randn(sa, generator=g).half()
    b = torch.randn(sb, generator=g).half()
    ref = mo.matmul(to_np(a), to_np(b), mode, mask, ta, tb)
    for _ in range(2):                                         # the second call reuses the stub's cached workspace
        c = ns["sparse_ops"].sparse_matmul(a.cuda(), b.cuda(), mode, layout.row_layout, layout.col_layout, ta, tb)
        assert tuple(c.shape) == ref.shape
        assert rel_err(to_np(c), ref) <= tol_of(torch.float16)
