"""GPU: configuration 5, SDD(QK^T) -> softmax -> DSD(PV) at batch 4 x 12 heads x seq 8192."""
import numpy as np
import pytest
import torch

from oracle import matmul_oracle as mo, softmax_oracle as so
from helpers import rel_err, to_np

pytestmark = pytest.mark.gpu


def test_config5_chain_fp16():
    import sparse, workloads as wl
    cfg = wl.config5()
    L = sparse.SparseLayout(cfg["mask"])
    assert L.num_blocks == 2526                       # seeded mask, see tests/golden/layout_tables.json
    q, k, v = (cfg[n].cuda() for n in ("q", "k", "v"))
    s = sparse.matmul(q, k, "sdd", L, False, True)
    p = sparse.softmax(s, L, cfg["scale"], cfg["causal"])
    o = sparse.matmul(p, v, "dsd", L)
    assert tuple(s.shape) == (4, 12, 2526, 32, 32) and tuple(o.shape) == (4, 12, 8192, 64)

    # float64 oracle, stage by stage, on one head (an 8192 x 8192 double matrix is 512 MB)
    m = cfg["mask"].numpy()
    b, h = 2, 7
    s_ref = mo.matmul(to_np(cfg["q"][b, h][None]), to_np(cfg["k"][b, h][None]), "sdd", m, False, True)
    assert rel_err(to_np(s[b, h][None]), s_ref) <= 2e-3
    p_ref = so.forward(to_np(s[b, h][None]), m, cfg["scale"], False)
    assert rel_err(to_np(p[b, h][None]), p_ref) <= 2e-3
    o_ref = mo.matmul(to_np(p[b, h][None]), to_np(cfg["v"][b, h][None]), "dsd", m)
    assert rel_err(to_np(o[b, h][None]), o_ref) <= 2e-3

    # every head against dense masked attention in fp32 torch on the GPU, end to end
    big = cfg["mask"].bool().cuda().repeat_interleave(32, 0).repeat_interleave(32, 1)
    worst = 0.0
    for bi in range(4):
        for hi in range(0, 12, 3):
            sc = (q[bi, hi].float() @ k[bi, hi].float().t()) * cfg["scale"]
            ref = torch.softmax(sc.masked_fill(~big, float("-inf")), -1) @ v[bi, hi].float()
            worst = max(worst, ((o[bi, hi].float() - ref).abs().max() / ref.abs().max()).item())
    assert worst <= 4e-3      # three fp16 roundings in a row (scores, probabilities, output)

    # rows of p sum to one on every head
    sums = torch.zeros(4, 12, 8192, device="cuda")
    rows = L.sparse_positions[:, 0]
    sums.view(4, 12, 256, 32).index_add_(2, rows, p.float().sum(-1))
    assert torch.allclose(sums, torch.ones_like(sums), atol=5e-3)


def test_split_groups_under_graph_capture():
    """Operators whose long groups meet in a workspace, captured into a HIP graph on another stream than
    the eager warm-up ran on: the capture takes the buffer the warm-up zeroed for it; every replay, with
    eager launches in between, gives the eager result.  A first use under capture is refused."""
    import sparse
    from sparse import _ops
    mask = np.zeros((130, 130), dtype=np.int64)
    mask[np.arange(130), np.arange(130)] = 1
    mask[:, 7] = 1                      # a column of 130 blocks: DDS splits it
    mask[9, :] = 1                      # a row of 130 blocks: DSD and the attention walks split it
    L = sparse.SparseLayout(torch.as_tensor(mask))
    g = torch.Generator().manual_seed(3)
    q, k, v = ((0.5 * torch.randn(2, 32 * 130, 64, generator=g)).half().cuda() for _ in range(3))
    w = (0.1 * torch.randn(2, L.num_blocks, 32, 32, generator=g)).half().cuda()

    def run():
        return (sparse.matmul(v, w, "dds", L, True, False), sparse.matmul(w, v, "dsd", L),
                sparse.attention(q, k, v, L, 0.125, True))
    with torch.no_grad():
        eager = run()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            captured = run()
        for _ in range(3):
            graph.replay()
            torch.cuda.synchronize()
            for a, b in zip(captured, eager):
                assert torch.equal(a, b)
            again = run()                                   # eager work between the replays
            for a, b in zip(again, eager):
                assert torch.equal(a, b)
