"""Loader of the HIP library and the ``sparse_ops`` boundary object.

Takes the place of ``sparse/kernel.py:6-16`` of the reference, which JIT-builds a
torch C++/CUDA extension at import time.  Here a prebuilt C-ABI shared object
(``csrc/libbsa_hip.so``, made by ``csrc/build.py`` with hipcc for gfx950) is
opened with ctypes; torch tensors cross the boundary as raw device pointers and
the current HIP stream.  If the library is missing the import fails loudly:
there is no fallback path.
"""
import ctypes
import os

import torch  # noqa: F401  (loads the HIP runtime the library binds to)

_CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
LIBRARY_PATH = os.path.join(_CSRC, "libbsa_hip.so")

BSA_F32, BSA_F16, BSA_BF16 = 0, 1, 2
BSA_SDD, BSA_DSD, BSA_DDS = 0, 1, 2
BSA_OK, BSA_ERR_INVALID, BSA_ERR_LAUNCH, BSA_ERR_UNSUPPORTED = 0, -1, -2, -3
MODES = {"sdd": BSA_SDD, "dsd": BSA_DSD, "dds": BSA_DDS}

_vp, _i, _i64, _f = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float

# name -> (restype, argtypes); mirrors include/bsa.h one to one
SIGNATURES = {
    "bsa_version": (_i, []),
    "bsa_last_error": (ctypes.c_char_p, []),
    "bsa_layout_workspace_bytes": (ctypes.c_size_t, [_i, _i]),
    "bsa_layout_build": (_i, [_vp, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "bsa_schedule_capacity": (_i64, [_i, _i, _i, _i]),
    "bsa_schedule_build": (_i, [_vp, _i, _i, _i, _i, _i, _i, _vp, _i64, _vp, _vp]),
    "bsa_matmul_workspace_bytes": (ctypes.c_size_t, [_i, _i, _i, _i, _i, _i]),
    "bsa_matmul": (_i, [_i, _i, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i, _vp, ctypes.c_size_t,
                        _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "bsa_matmul_noalloc": (_i, [_i, _i, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i,
                                _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "bsa_matmul_dsd_block64": (_i, [_i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "bsa_run_schedule_bytes": (ctypes.c_int64, [_i, _i]),
    "bsa_run_schedule_build": (_i, [_vp, _vp, _i, _i, _i, _i, _vp, ctypes.c_int64, _vp, _vp]),
    "bsa_matmul_dsd_runs": (_i, [_i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "bsa_softmax_forward": (_i, [_i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _i, _vp]),
    "bsa_softmax_backward": (_i, [_i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _vp]),
    "bsa_to_sparse": (_i, [_i, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "bsa_to_dense": (_i, [_i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "bsa_attention_workspace_bytes": (ctypes.c_size_t, [_i, _i, _i, _i]),
    "bsa_attention_forward": (_i, [_i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, ctypes.c_size_t,
                                   _i, _i, _i, _i, _i, _f, _i, _vp]),
    "bsa_attention_backward_workspace_bytes": (ctypes.c_size_t, [_i, _i, _i, _i, _i, _i]),
    "bsa_attention_backward_scores": (_i, [_i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i,
                                           _i, _i, _vp, ctypes.c_size_t, _i, _i, _i, _i, _i, _f, _i, _vp]),
    "bsa_attention_backward": (_i, [_i] + [_vp] * 10 + [_vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _vp, _i, _i, _i, _i,
                                                        _vp, ctypes.c_size_t, _i, _i, _i, _i, _i, _f, _i, _vp]),
}


class BsaError(RuntimeError):
    """A C-ABI call returned a nonzero status."""


def load_library(path: str = LIBRARY_PATH) -> ctypes.CDLL:
    if not os.path.exists(path):
        raise ImportError(
            f"{path} is missing: build it with `python {os.path.join(_CSRC, 'build.py')}` "
            "(hipcc, --offload-arch=gfx950). There is no fallback implementation.")
    lib = ctypes.CDLL(path)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)      # AttributeError if the symbol is not exported
        fn.restype, fn.argtypes = restype, argtypes
    return lib


lib = load_library()


def check(status: int) -> None:
    if status != 0:
        raise BsaError(f"bsa status {status}: {lib.bsa_last_error().decode()}")


def current_stream() -> int:
    return torch.cuda.current_stream().cuda_stream


from . import _ops as sparse_ops  # noqa: E402  (module with the reference's sparse_matmul signature)
