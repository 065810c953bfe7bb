"""Block masks and seeded synthetic inputs of the five benchmark configurations.

Everything is drawn on the CPU from ``torch.Generator().manual_seed(1000 + n)``
in a fixed order, in float32, then cast, so the GPU run, the CPU baseline and
the parity tests see identical bits.  Shapes follow the configuration list:

1  SDD  fp32  A[1,512,64] x B[1,512,64]^T on a 16x16 Bernoulli(0.25)+diagonal mask
2  DSD  fp16  S[16,314,32,32] (row-normalised U(0,1), +-2 block window, 2048^2) x B[16,2048,64]
3  softmax fp16  X[16,1530,32,32] ~ N(0,4), seq 4096, causal local-4 + every-8th-column mask,
                 scale 1/8, causal
4  DDS  fp16  dY[16,4096,64]^T x W[16,1530,32,32] (N(0,0.02)), same mask as 3 -> [16,64,4096]
5  chain fp16 Q,K,V[4,12,8192,64]: SDD(QK^T) -> softmax(1/8) -> DSD(PV) on a BigBird-style mask
"""
import torch

BLOCK = 32


def mask_random_diag(n: int, density: float, gen: torch.Generator) -> torch.Tensor:
    return ((torch.rand(n, n, generator=gen) < density) | torch.eye(n, dtype=torch.bool)).long()


def mask_local_window(n: int, radius: int) -> torch.Tensor:
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    return ((i - j).abs() <= radius).long()


def mask_causal_local_strided(n: int, window: int = 4, stride: int = 8) -> torch.Tensor:
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    return ((j <= i) & ((i - j < window) | (j % stride == 0))).long()


def mask_bigbird(n: int, gen: torch.Generator, radius: int = 1, n_global: int = 2,
                 n_random: int = 3) -> torch.Tensor:
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    mask = ((i - j).abs() <= radius) | (i < n_global) | (j < n_global)
    rnd = torch.randint(0, n, (n, n_random), generator=gen)
    mask = mask.clone()
    mask[torch.arange(n)[:, None].expand(n, n_random), rnd] = True
    return mask.long()


def _gen(config: int) -> torch.Generator:
    return torch.Generator().manual_seed(1000 + config)


def dense_of(mask: torch.Tensor) -> torch.Tensor:
    """Element-level 0/1 mask of a block mask."""
    return mask.repeat_interleave(BLOCK, 0).repeat_interleave(BLOCK, 1)


def blocks_of(mask: torch.Tensor, dense: torch.Tensor) -> torch.Tensor:
    """``[..., R*32, C*32]`` -> ``[..., nnz, 32, 32]`` on the CPU (row-major block order)."""
    rows, cols = mask.shape
    pos = torch.nonzero(mask)
    tiles = dense.reshape(dense.shape[:-2] + (rows, BLOCK, cols, BLOCK)).transpose(-3, -2)
    tiles = tiles.reshape(dense.shape[:-2] + (rows * cols, BLOCK, BLOCK))
    return tiles.index_select(-3, pos[:, 0] * cols + pos[:, 1]).contiguous()


def config1():
    g = _gen(1)
    mask = mask_random_diag(16, 0.25, g)
    a = torch.randn(1, 512, 64, generator=g)
    b = torch.randn(1, 512, 64, generator=g)
    return {"mask": mask, "a": a, "b": b, "mode": "sdd", "trans_a": False, "trans_b": True,
            "dtype": torch.float32}


def config2(batch: int = 16):
    g = _gen(2)
    mask = mask_local_window(64, 2)
    dm = dense_of(mask).float()
    s = torch.empty(batch, int(mask.sum()), BLOCK, BLOCK)
    for i in range(batch):                      # one head at a time keeps the peak at 2048^2 floats
        d = torch.rand(2048, 2048, generator=g) * dm
        d /= d.sum(-1, keepdim=True)
        s[i] = blocks_of(mask, d)
    b = torch.randn(batch, 2048, 64, generator=g)
    return {"mask": mask, "a": s.half(), "b": b.half(), "mode": "dsd", "trans_a": False,
            "trans_b": False, "dtype": torch.float16}


def config3(batch: int = 16):
    g = _gen(3)
    mask = mask_causal_local_strided(128)
    nnz = int(mask.sum())
    x = 2.0 * torch.randn(batch, nnz, BLOCK, BLOCK, generator=g)
    return {"mask": mask, "x": x.half(), "scale": 0.125, "causal": True, "dtype": torch.float16}


def config4(batch: int = 16):
    g = _gen(4)
    mask = mask_causal_local_strided(128)
    nnz = int(mask.sum())
    dy = torch.randn(batch, 4096, 64, generator=g)
    w = 0.02 * torch.randn(batch, nnz, BLOCK, BLOCK, generator=g)
    return {"mask": mask, "a": dy.half(), "b": w.half(), "mode": "dds", "trans_a": True,
            "trans_b": False, "dtype": torch.float16}


def config5(batch: int = 4, heads: int = 12, seq: int = 8192):
    g = _gen(5)
    mask = mask_bigbird(seq // BLOCK, g)
    q = torch.randn(batch, heads, seq, 64, generator=g)
    k = torch.randn(batch, heads, seq, 64, generator=g)
    v = torch.randn(batch, heads, seq, 64, generator=g)
    return {"mask": mask, "q": q.half(), "k": k.half(), "v": v.half(), "scale": 0.125,
            "causal": False, "dtype": torch.float16}


def seq4096(batch: int = 16, head_dim: int = 64, seed: int = 1004):
    """The seq-4096 / block-32 / ~10 % density workload the headline metric is quoted on:
    one attention-shaped set of operands on the configuration-3/4 mask."""
    g = torch.Generator().manual_seed(seed)
    mask = mask_causal_local_strided(128)
    nnz = int(mask.sum())
    q = torch.randn(batch, 4096, head_dim, generator=g).half()
    k = torch.randn(batch, 4096, head_dim, generator=g).half()
    v = torch.randn(batch, 4096, head_dim, generator=g).half()
    scores = (2.0 * torch.randn(batch, nnz, BLOCK, BLOCK, generator=g)).half()
    w = (0.02 * torch.randn(batch, nnz, BLOCK, BLOCK, generator=g)).half()
    return {"mask": mask, "q": q, "k": k, "v": v, "scores": scores, "w": w, "scale": 0.125}
