"""CPU: the table oracle against known answers, brute force, the C walk and invariants."""
import json
import os

import numpy as np
import pytest
from hypothesis import given, settings, strategies as st

from oracle import c_oracle, layout_oracle as lo
from helpers import mask_zoo

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def test_known_answer_3x3():
    # derived by hand from the definition (row-major ordinal, (row << 16) + col)
    mask = np.array([[1, 0, 1], [0, 1, 0], [1, 1, 0]])
    rb, ro = lo.create_layout(mask)
    cb, co = lo.create_layout(mask, transpose=True)
    assert rb.tolist() == [0, 0, 1, 2, 2, 65537, 3, 131072, 4, 131073]
    assert ro.tolist() == [0, 2, 3, 5]
    assert cb.tolist() == [0, 0, 3, 131072, 2, 65537, 4, 131073, 1, 2]
    assert co.tolist() == [0, 2, 4, 5]
    assert rb.dtype == np.int32 and ro.dtype == np.int32


@pytest.mark.parametrize("name,mask", mask_zoo())
@pytest.mark.parametrize("transpose", [False, True])
def test_three_builders_agree(name, mask, transpose):
    b1, o1 = lo.create_layout(mask, transpose)
    b2, o2 = lo.create_layout_bruteforce(mask, transpose)
    b3, o3 = c_oracle.layout(mask, transpose)
    assert np.array_equal(b1, b2) and np.array_equal(o1, o2)
    assert np.array_equal(b1, b3) and np.array_equal(o1, o3)


def _check_invariants(mask):
    nnz = int(np.count_nonzero(mask))
    rb, ro = lo.create_layout(mask)
    cb, co = lo.create_layout(mask, transpose=True)
    for blocks, offs, groups in ((rb, ro, mask.shape[0]), (cb, co, mask.shape[1])):
        assert len(blocks) == 2 * nnz and len(offs) == groups + 1
        assert offs[0] == 0 and offs[-1] == nnz and np.all(np.diff(offs) >= 0)
        idx, r, c = lo.decode_blocks(blocks)
        assert sorted(idx.tolist()) == list(range(nnz))           # idx is a permutation
        assert np.all(mask[r, c] != 0)
    # row and column tables hold the same (idx, pos) pairs
    assert sorted(map(tuple, rb.reshape(-1, 2).tolist())) == sorted(map(tuple, cb.reshape(-1, 2).tolist()))
    # groups really group
    idx, r, c = lo.decode_blocks(rb)
    for g in range(mask.shape[0]):
        assert np.all(r[ro[g]:ro[g + 1]] == g) and np.all(np.diff(c[ro[g]:ro[g + 1]]) > 0)
    idx, r, c = lo.decode_blocks(cb)
    for g in range(mask.shape[1]):
        assert np.all(c[co[g]:co[g + 1]] == g) and np.all(np.diff(r[co[g]:co[g + 1]]) > 0)


@pytest.mark.parametrize("name,mask", mask_zoo())
def test_invariants(name, mask):
    _check_invariants(np.asarray(mask))


@settings(max_examples=40, deadline=None)
@given(st.integers(1, 40), st.integers(1, 40), st.floats(0.0, 1.0), st.integers(0, 2 ** 31 - 1))
def test_invariants_random(rows, cols, density, seed):
    mask = (np.random.RandomState(seed).rand(rows, cols) < density).astype(np.int64)
    _check_invariants(mask)
    b1, o1 = lo.create_layout(mask, True)
    b2, o2 = lo.create_layout_bruteforce(mask, True)
    assert np.array_equal(b1, b2) and np.array_equal(o1, o2)


def test_bool_and_int_masks_mean_the_same():
    mask = np.array([[1, 0, 1], [0, 1, 0], [1, 1, 0]])
    for tr in (False, True):
        a = lo.create_layout(mask, tr)
        b = lo.create_layout(mask.astype(bool), tr)
        c = lo.create_layout(mask * 5, tr)      # any nonzero marks a block
        assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
        assert np.array_equal(a[0], c[0]) and np.array_equal(a[1], c[1])


def test_wide_mask_decodes_16_bit_columns():
    mask = np.zeros((2, 300), dtype=np.int64)
    mask[1, 299] = 1
    mask[0, 256] = 1
    blocks, _ = lo.create_layout(mask)
    _, r, c = lo.decode_blocks(blocks)
    assert r.tolist() == [0, 1] and c.tolist() == [256, 299]


@pytest.mark.parametrize("name,mask", mask_zoo())
def test_to_sparse_to_dense_roundtrip(name, mask):
    mask = np.asarray(mask)
    rng = np.random.RandomState(0)
    x = rng.randn(2, mask.shape[0] * 32, mask.shape[1] * 32)
    s = lo.to_sparse(mask, x)
    assert s.shape == (2, int(np.count_nonzero(mask)), 32, 32)
    d = lo.to_dense(mask, s, 0.0)
    big = np.kron(mask != 0, np.ones((32, 32)))
    assert np.array_equal(d, x * big)
    assert np.array_equal(lo.to_sparse(mask, d), s)
    dinf = lo.to_dense(mask, s, -np.inf)
    assert np.all(np.isneginf(dinf[:, big == 0]))


def test_golden_tables():
    """Tables of the five benchmark masks, as committed by tests/golden/make_golden.py."""
    with open(os.path.join(GOLDEN, "layout_tables.json")) as f:
        golden = json.load(f)
    import workloads as wl
    masks = {
        "config1": wl.config1()["mask"].numpy(),
        "config2": wl.mask_local_window(64, 2).numpy(),
        "config3_4": wl.mask_causal_local_strided(128).numpy(),
        "config5": wl.mask_bigbird(256, wl._gen(5)).numpy(),
    }
    for name, mask in masks.items():
        g = golden[name]
        assert int(np.count_nonzero(mask)) == g["nnz"], name
        for tr, key in ((False, "row"), (True, "col")):
            blocks, offs = lo.create_layout(mask, tr)
            assert offs.tolist() == g[key + "_offsets"], name
            assert int(blocks.astype(np.int64).sum()) == g[key + "_blocks_sum"], name
            assert blocks[:16].tolist() == g[key + "_blocks_head"], name
            # position-weighted checksum: catches reorderings the plain sum misses
            w = np.arange(1, len(blocks) + 1, dtype=np.int64)
            assert int((blocks.astype(np.int64) * w % 1000003).sum()) == g[key + "_blocks_wsum"], name
