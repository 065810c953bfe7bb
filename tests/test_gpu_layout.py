"""GPU: the device table builder is bit-exact with the oracle; schedules are valid."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import layout_oracle as lo
from helpers import mask_zoo

pytestmark = pytest.mark.gpu


def _layout(mask):
    import sparse
    return sparse.SparseLayout(torch.as_tensor(np.asarray(mask)))


def _more_masks():
    rng = np.random.RandomState(11)
    out = list(mask_zoo())
    out.append(("rand_256x256", (rng.rand(256, 256) < 0.1).astype(np.int64)))
    out.append(("rand_100x37", (rng.rand(100, 37) < 0.5).astype(np.int64)))
    out.append(("empty_33x65", np.zeros((33, 65), dtype=np.int64)))
    out.append(("full_40x40", np.ones((40, 40), dtype=np.int64)))
    wide = np.zeros((3, 300), dtype=np.int64)
    wide[0, 256] = wide[1, 299] = wide[2, 0] = 1
    out.append(("wide_3x300", wide))
    return out


@pytest.mark.parametrize("name,mask", _more_masks())
def test_tables_bit_exact(name, mask):
    mask = np.asarray(mask)
    L = _layout(mask)
    for tr, got in ((False, L.row_layout), (True, L.col_layout)):
        blocks, offs = lo.create_layout(mask, tr)
        assert got[0].dtype == torch.int32 and got[1].dtype == torch.int32 and got[0].is_cuda
        assert np.array_equal(got[0].cpu().numpy(), blocks), (name, tr)
        assert np.array_equal(got[1].cpu().numpy(), offs), (name, tr)
    assert np.array_equal(L.sparse_positions.cpu().numpy(), lo.sparse_positions(mask))


def test_bool_and_scaled_masks():
    mask = np.array([[1, 0, 1], [0, 1, 0], [1, 1, 0]])
    ref = lo.create_layout(mask)
    for m in (torch.as_tensor(mask).bool(), torch.as_tensor(mask * 3), torch.as_tensor(mask).float()):
        import sparse
        L = sparse.SparseLayout(m)
        assert np.array_equal(L.row_layout[0].cpu().numpy(), ref[0])
        assert np.array_equal(L.row_layout[1].cpu().numpy(), ref[1])


def test_golden_tables_on_device():
    import workloads as wl
    with open(os.path.join(os.path.dirname(__file__), "golden", "layout_tables.json")) as f:
        golden = json.load(f)
    masks = {"config1": wl.config1()["mask"], "config2": wl.mask_local_window(64, 2),
             "config3_4": wl.mask_causal_local_strided(128), "config5": wl.mask_bigbird(256, wl._gen(5))}
    for name, mask in masks.items():
        L = _layout(mask.numpy())
        g = golden[name]
        assert L.num_blocks == g["nnz"]
        for key, got in (("row", L.row_layout), ("col", L.col_layout)):
            blocks = got[0].cpu().numpy().astype(np.int64)
            w = np.arange(1, len(blocks) + 1, dtype=np.int64)
            assert got[1].cpu().tolist() == g[key + "_offsets"]
            assert int(blocks.sum()) == g[key + "_blocks_sum"]
            assert int((blocks * w % 1000003).sum()) == g[key + "_blocks_wsum"]


@pytest.mark.parametrize("name,mask", _more_masks())
@pytest.mark.parametrize("longest", [False, True])
@pytest.mark.parametrize("cap,waves,split", [(4, 8, True), (1, 4, True), (16, 2, True), (3, 1, True),
                                             (4, 8, False), (2, 2, False)])
def test_schedule_covers_every_pair_once(name, mask, cap, waves, split, longest):
    from sparse import _ops
    mask = np.asarray(mask)
    L = _layout(mask)
    for layout in (L.row_layout, L.col_layout):
        offs = layout[1].cpu().numpy()
        groups = len(offs) - 1
        s = _ops.Schedule(layout[1], layout[0].numel() // 2, cap, waves, split, longest_first=longest)
        raw = s.table.cpu().numpy().reshape(-1, 4)
        meta = raw[:groups]
        tab = raw[groups: groups + s.workgroups * waves]
        assert s.slots <= s.workgroups * waves
        seen = np.zeros(max(int(offs[-1]), 1), dtype=np.int64)
        parts_seen = [set() for _ in range(groups)]
        tile_slots = split_groups = 0
        for slot, (g, b, e, team) in enumerate(tab):
            if g < 0:
                continue
            team = int(team) & 0xFFFFFFFF
            first, nw, part, parts = team & 0xF, (team >> 4) & 0xF, (team >> 8) & 0xFFF, team >> 20
            wg, in_wg = divmod(slot, waves)
            assert 0 <= g < groups and offs[g] <= b <= e <= offs[g + 1]
            assert first <= in_wg < first + nw <= waves            # a team sits inside one workgroup
            assert parts == meta[g][3] and 0 <= part < parts
            leader = tab[wg * waves + first]
            assert leader[0] == g and leader[3] == tab[slot][3]
            seen[b:e] += 1
            if in_wg == first:
                assert part not in parts_seen[g]
                parts_seen[g].add(part)
                chunks = tab[wg * waves + first: wg * waves + first + nw]
                assert all(chunks[i][2] == chunks[i + 1][1] for i in range(nw - 1))   # consecutive
                plen = chunks[-1][2] - chunks[0][1]
                assert nw == min(max(-(-plen // cap), 1), waves)
                if split:
                    assert plen <= cap * waves
                if part == 0:
                    assert chunks[0][1] == offs[g] and meta[g][0] == slot
                if part == parts - 1:
                    assert chunks[-1][2] == offs[g + 1]
        assert np.all(seen[: int(offs[-1])] == 1)
        if longest:
            # unsplit groups sit in the order of their longest chunk's class (quarters of cap), longest first
            classes = []
            for slot, (g, b, e, team) in enumerate(tab):
                team = int(team) & 0xFFFFFFFF
                if g < 0 or (team >> 20) != 1 or slot % waves != (team & 0xF):
                    continue
                nw, length = (team >> 4) & 0xF, offs[g + 1] - offs[g]
                chunk = -(-length // nw)
                classes.append(0 if 4 * chunk > 3 * cap else 1 if 2 * chunk > cap else 2 if 4 * chunk > cap else 3)
            assert classes == sorted(classes)
        for g in range(groups):
            length = offs[g + 1] - offs[g]
            want = max(-(-length // (cap * waves)), 1) if split else 1
            assert parts_seen[g] == set(range(want)), (g, parts_seen[g], want)   # empty groups get a slot too
            if want > 1:
                assert meta[g][1] == tile_slots and meta[g][2] == split_groups
                tile_slots += want
                split_groups += 1
            else:
                assert meta[g][1] == -1 and meta[g][2] == -1
        assert (s.tile_slots, s.split_groups) == (tile_slots, split_groups)


@pytest.mark.parametrize("name,mask", _more_masks())
@pytest.mark.parametrize("longest", [False, True])
@pytest.mark.parametrize("cap,waves,slice_max,slices", [(4, 4, 24, 2), (4, 4, 3, 4), (2, 2, 0, 2), (4, 8, 64, 4), (4, 8, 24, 8)])
def test_row_sliced_schedule(name, mask, cap, waves, slice_max, slices, longest):
    """Softmax schedules with slice_max: a short row goes whole to `slices` wavefronts (one slice of
    its element rows each) that sit among other sliced rows at the front of the schedule; every
    other row is chunked as without slicing and never split into parts.  Longest first, the sliced
    rows come behind the others, by quarters of the longest sliced row's length and in table order
    inside a quarter."""
    from sparse import _ops
    mask = np.asarray(mask)
    L = _layout(mask)
    offs = L.row_layout[1].cpu().numpy()
    groups = len(offs) - 1
    s = _ops.Schedule(L.row_layout[1], L.num_blocks, cap, waves, False, slice_max, slices, longest_first=longest)
    raw = s.table.cpu().numpy().reshape(-1, 4)
    meta, tab = raw[:groups], raw[groups: groups + s.workgroups * waves]
    assert (s.tile_slots, s.split_groups) == (0, 0)
    sliced = [g for g in range(groups) if offs[g + 1] - offs[g] <= slice_max]
    slices_seen = {g: [] for g in sliced}
    covered = np.zeros(max(int(offs[-1]), 1), dtype=np.int64)
    last_sliced_wg, first_other_wg = -1, s.workgroups
    first_sliced_wg, last_other_wg = s.workgroups, -1
    for slot, (g, b, e, team) in enumerate(tab):
        if g < 0:
            continue
        team = int(team) & 0xFFFFFFFF
        first, nw, part, parts = team & 0xF, (team >> 4) & 0xF, (team >> 8) & 0xFFF, team >> 20
        wg, in_wg = divmod(slot, waves)
        if g in slices_seen:
            assert (b, e) == (offs[g], offs[g + 1]) and nw == 1 and parts == slices and first == in_wg
            slices_seen[g].append((wg, part))
            last_sliced_wg = max(last_sliced_wg, wg)
            first_sliced_wg = min(first_sliced_wg, wg)
        else:
            assert parts == 1 and part == 0 and first <= in_wg < first + nw <= waves
            covered[b:e] += 1
            first_other_wg = min(first_other_wg, wg)
            last_other_wg = max(last_other_wg, wg)
            assert meta[g][0] == groups * 0 + (wg * waves + first)
    for g in sliced:
        got = sorted(slices_seen[g])
        assert sorted(p for _, p in got) == list(range(slices)), (g, got)            # every slice once
        covered[offs[g]: offs[g + 1]] += 1
    assert np.all(covered[: int(offs[-1])] == 1)
    if longest:                                                 # sliced rows fill workgroups of their own: behind the
        assert last_other_wg < first_sliced_wg                  # longer rows when long work goes first, else in front
    else:
        assert last_sliced_wg < first_other_wg
    order = [int(g) for slot, (g, b, e, team) in enumerate(tab) if g in slices_seen and ((int(team) >> 8) & 0xFFF) == 0]
    assert sorted(order) == sorted(sliced)
    if longest and sliced:
        yard = max(offs[g + 1] - offs[g] for g in sliced)
        quarter = lambda n: 0 if 4 * n > 3 * yard else 1 if 2 * n > yard else 2 if 4 * n > yard else 3
        assert order == sorted(sliced, key=lambda g: (quarter(offs[g + 1] - offs[g]), g))
    else:
        assert order == sliced


@pytest.mark.parametrize("name,mask", _more_masks())
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.float64])
def test_to_sparse_to_dense_on_device(name, mask, dtype):
    """fp16 / fp32 go through the copy kernels, float64 through the torch gather: both must equal the
    slice definition, and to_dense must write zeros where no block is stored."""
    mask = np.asarray(mask)
    if mask.size > 4096:
        pytest.skip("dense matrix too large for a quick test")
    L = _layout(mask)
    r, c = mask.shape
    g = torch.Generator().manual_seed(r * 131 + c)
    x = torch.randn(2, 3, 32 * r, 32 * c, generator=g).to(dtype)
    s = L.to_sparse(x.cuda())
    assert s.dtype == dtype and tuple(s.shape) == (2, 3, L.num_blocks, 32, 32)
    assert np.array_equal(s.cpu().numpy(), lo.to_sparse(mask, x.numpy()))
    d = L.to_dense(s)
    assert tuple(d.shape) == tuple(x.shape)
    assert np.array_equal(d.cpu().numpy(), lo.to_dense(mask, lo.to_sparse(mask, x.numpy()), 0.0))
    # no batch dimension, and a non-contiguous view
    assert np.array_equal(L.to_sparse(x[0, 1].cuda()).cpu().numpy(), lo.to_sparse(mask, x[0, 1].numpy()))
    xt = x.cuda().transpose(0, 1)
    assert np.array_equal(L.to_sparse(xt).cpu().numpy(), lo.to_sparse(mask, xt.cpu().numpy()))


def test_to_sparse_to_dense_gradients():
    mask = np.asarray(dict(mask_zoo())["rand16"])
    L = _layout(mask)
    x = torch.randn(2, 512, 512, device="cuda", requires_grad=True)
    w = torch.randn(2, L.num_blocks, 32, 32, device="cuda")
    (L.to_sparse(x) * w).sum().backward()
    assert torch.equal(x.grad, L.to_dense(w))                   # gradient of a gather is the scatter, zeros elsewhere
    s = torch.randn(2, L.num_blocks, 32, 32, device="cuda", requires_grad=True)
    u = torch.randn(2, 512, 512, device="cuda")
    (L.to_dense(s) * u).sum().backward()
    assert torch.equal(s.grad, L.to_sparse(u))
