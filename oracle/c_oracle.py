"""ctypes front end of ``bsa_oracle.c`` (TEST INFRASTRUCTURE ONLY).

Arrays go in as float32 (fp16 data widened exactly), results come back as
float64.  ``load()`` builds the shared object with ``make`` when it is missing.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

_f32 = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_f64 = np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS")
_i32 = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
_u8 = np.ctypeslib.ndpointer(np.uint8, flags="C_CONTIGUOUS")
_int, _dbl = ctypes.c_int, ctypes.c_double


def build(force: bool = False) -> str:
    path = os.path.join(_HERE, "libbsa_oracle.so")
    if force or not os.path.exists(path):
        subprocess.run(["make", "-B" if force else "-s", "-C", _HERE, "libbsa_oracle.so"],
                       check=True, capture_output=True)
    return path


def load():
    global _LIB
    if _LIB is None:
        lib = ctypes.CDLL(build())
        lib.bsa_oracle_layout.argtypes = [_u8, _int, _int, _int, _i32, _i32]
        lib.bsa_oracle_layout.restype = _int
        lib.bsa_oracle_sdd.argtypes = [_f32, _f32, _f64, _i32] + [_int] * 7
        lib.bsa_oracle_dsd.argtypes = [_f32, _f32, _f64, _i32, _i32] + [_int] * 7
        lib.bsa_oracle_dds.argtypes = [_f32, _f32, _f64, _i32, _i32] + [_int] * 7
        lib.bsa_oracle_softmax_fwd.argtypes = [_f32, _f64, _i32, _i32, _int, _int, _int, _dbl, _int]
        lib.bsa_oracle_softmax_bwd.argtypes = [_f32, _f32, _f64, _i32, _i32, _int, _int, _int, _dbl]
        for f in ("sdd", "dsd", "dds", "softmax_fwd", "softmax_bwd"):
            getattr(lib, "bsa_oracle_" + f).restype = None
        _LIB = lib
    return _LIB


def _f(x):
    return np.ascontiguousarray(np.asarray(x, dtype=np.float32))


def layout(pattern, transpose=False):
    mask = np.ascontiguousarray((np.asarray(pattern) != 0).astype(np.uint8))
    R, C = mask.shape
    blocks = np.zeros(2 * R * C, dtype=np.int32)
    offsets = np.zeros((C if transpose else R) + 1, dtype=np.int32)
    nnz = load().bsa_oracle_layout(mask, R, C, int(transpose), blocks, offsets)
    return blocks[:2 * nnz].copy(), offsets


def matmul(a, b, mode, pattern, trans_a=False, trans_b=False):
    """Block-walk product; batch dims are flattened like sparse_kernels.cc:29-30."""
    lib = load()
    a, b = _f(a), _f(b)
    row = layout(pattern, False)
    col = layout(pattern, True)
    nnz = len(row[0]) // 2
    if mode == "sdd":
        batch = a.shape[:-2]
        M = a.shape[-1] if trans_a else a.shape[-2]
        K = a.shape[-2] if trans_a else a.shape[-1]
        N = b.shape[-2] if trans_b else b.shape[-1]
        nb = int(np.prod(batch, dtype=np.int64))
        c = np.zeros((nb, nnz, 32, 32), dtype=np.float64)
        lib.bsa_oracle_sdd(a.reshape(nb, -1), b.reshape(nb, -1), c, row[0], nnz, nb, M, N, K,
                           int(trans_a), int(trans_b))
        return c.reshape(batch + (nnz, 32, 32))
    if mode == "dsd":
        blocks, offs = row if not trans_a else col
        batch = b.shape[:-2]
        K = b.shape[-1] if trans_b else b.shape[-2]
        N = b.shape[-2] if trans_b else b.shape[-1]
        groups = len(offs) - 1
        nb = int(np.prod(batch, dtype=np.int64))
        c = np.zeros((nb, groups * 32, N), dtype=np.float64)
        lib.bsa_oracle_dsd(a.reshape(nb, -1), b.reshape(nb, -1), c, blocks, offs, groups, nnz, nb,
                           N, K, int(trans_a), int(trans_b))
        return c.reshape(batch + (groups * 32, N))
    if mode == "dds":
        blocks, offs = col if not trans_b else row
        batch = a.shape[:-2]
        M = a.shape[-1] if trans_a else a.shape[-2]
        K = a.shape[-2] if trans_a else a.shape[-1]
        groups = len(offs) - 1
        nb = int(np.prod(batch, dtype=np.int64))
        c = np.zeros((nb, M, groups * 32), dtype=np.float64)
        lib.bsa_oracle_dds(a.reshape(nb, -1), b.reshape(nb, -1), c, blocks, offs, groups, nnz, nb,
                           M, K, int(trans_a), int(trans_b))
        return c.reshape(batch + (M, groups * 32))
    raise ValueError(mode)


def softmax_fwd(x, pattern, scale=1.0, causal=False):
    x = _f(x)
    blocks, offs = layout(pattern, False)
    nnz = len(blocks) // 2
    nb = x.size // max(nnz * 1024, 1) if nnz else 0
    y = np.zeros(x.shape, dtype=np.float64)
    if nnz:
        load().bsa_oracle_softmax_fwd(x.reshape(-1), y.reshape(-1), blocks, offs, len(offs) - 1,
                                      nnz, nb, float(scale), int(causal))
    return y


def softmax_bwd(y, dy, pattern, scale=1.0):
    y, dy = _f(y), _f(dy)
    blocks, offs = layout(pattern, False)
    nnz = len(blocks) // 2
    nb = y.size // max(nnz * 1024, 1) if nnz else 0
    dx = np.zeros(y.shape, dtype=np.float64)
    if nnz:
        load().bsa_oracle_softmax_bwd(y.reshape(-1), dy.reshape(-1), dx.reshape(-1), blocks, offs,
                                      len(offs) - 1, nnz, nb, float(scale))
    return dx
