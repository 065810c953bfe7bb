"""Masked-dense CPU baseline of the seq-4096 matmul workload (TEST/BENCH INFRASTRUCTURE ONLY).

The reported CPU figure is the dense meaning of the three products, run with
torch on the host cores in float32 on the fp16-rounded inputs:

    SDD  to_sparse(q @ k^T)       DSD  dense0(p) @ v       DDS  dy^T @ dense0(w)

on a bounded sample of heads.  It is a baseline to print next to the GPU
number, not a target.  Softmax: to_sparse(softmax(scale * dense_neginf(x) + causal)).
"""
import os
import time

import torch

BLOCK = 32


def _to_sparse(mask, dense):
    rows, cols = mask.shape
    pos = torch.nonzero(mask)
    t = dense.reshape(dense.shape[:-2] + (rows, BLOCK, cols, BLOCK)).transpose(-3, -2)
    t = t.reshape(dense.shape[:-2] + (rows * cols, BLOCK, BLOCK))
    return t.index_select(-3, pos[:, 0] * cols + pos[:, 1])


def _to_dense(mask, blocks, fill=0.0):
    rows, cols = mask.shape
    pos = torch.nonzero(mask)
    t = blocks.new_full(blocks.shape[:-3] + (rows * cols, BLOCK, BLOCK), fill)
    t.index_copy_(-3, pos[:, 0] * cols + pos[:, 1], blocks)
    t = t.reshape(blocks.shape[:-3] + (rows, cols, BLOCK, BLOCK)).transpose(-3, -2)
    return t.reshape(blocks.shape[:-3] + (rows * BLOCK, cols * BLOCK))


def matmul_step(mask, q, k, v, p, w):
    s = _to_sparse(mask, q @ k.transpose(-1, -2))
    o = _to_dense(mask, p) @ v
    g = v.transpose(-1, -2) @ _to_dense(mask, w)
    return s, o, g


def softmax_step(mask, x, scale, causal):
    d = _to_dense(mask, x * scale, float("-inf"))
    if causal:
        n = d.shape[-1]
        d = d.masked_fill(torch.triu(torch.ones(n, n, dtype=torch.bool), 1), float("-inf"))
    return _to_sparse(mask, torch.softmax(d, -1))


def time_seq4096(workload, heads: int = 2, repeats: int = 5):
    """Median wall time of the three masked-dense products and of the softmax on `heads` heads."""
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    mask = workload["mask"]
    q, k, v = (workload[n][:heads].float() for n in ("q", "k", "v"))
    p, w, x = (workload[n][:heads].float() for n in ("scores", "w", "scores"))
    out = {}
    for name, fn in (("matmul", lambda: matmul_step(mask, q, k, v, p, w)),
                     ("softmax", lambda: softmax_step(mask, x, workload["scale"], True))):
        fn()
        ts = []
        for _ in range(repeats):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        out[name] = sorted(ts)[len(ts) // 2]
    out["cores"] = cores
    out["heads"] = heads
    return out
