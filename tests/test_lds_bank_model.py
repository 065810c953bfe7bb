"""CPU: every LDS access map the kernels use, replayed through the CDNA4 bank model.

The addresses come from the host build of csrc/lds_index_math.hpp, the same functions the
device code calls, so a changed swizzle is checked without a GPU.
"""
import ctypes
import os

import pytest

import lds_bank_model as m


@pytest.mark.parametrize("name,width,variants", m.KERNEL_ACCESSES, ids=[a[0] for a in m.KERNEL_ACCESSES])
def test_kernel_accesses_are_conflict_free(name, width, variants):
    for kw in variants:
        addr = m.kernel_access(name, **kw)
        assert len(set(addr)) == 64 or name.startswith("get"), "two lanes write one slot"
        factor = m.KNOWN_COST_FACTOR.get(name, 1)     # 1: conflict-free; the exceptions are listed with their reason
        for model, banks in m.MODELS.items():
            assert m.access_cost(addr, width, banks) == factor * m.ideal_cost(width, banks), (name, kw, model)


def test_model_sees_the_conflicts_of_unswizzled_tiles():
    # one 16-byte piece of 32 rows of 64 bytes, no swizzle: rows r, r+4, r+8, r+12 collide (4-way)
    naive = [64 * (lane % 32) + 16 * (lane // 32) for lane in range(64)]
    assert m.access_cost(naive, 16, 64) == 4 * m.ideal_cost(16, 64)
    # the pad-by-one layout of the reference (33-float rows, sparse_smm_gpu.cu:29) is built for 32
    # lanes and 32 banks; read down a column by the 64 lanes of a wave it is a two-way conflict here,
    # and without the pad a 16-way one (128-byte rows, two rows per bank window)
    padded = [4 * (33 * (lane % 32) + lane // 32) for lane in range(64)]
    assert m.access_cost(padded, 4, 64) == 2
    unpadded = [4 * (32 * (lane % 32) + lane // 32) for lane in range(64)]
    assert m.access_cost(unpadded, 4, 64) == 16
    # linear accesses are the yardstick
    for width in (4, 8, 16):
        assert m.conflict_free([width * lane for lane in range(64)], width)


def test_swizzled_tiles_hold_every_element_once():
    """put followed by get returns the tile: the write and read maps agree (no aliasing)."""
    for permuted in (False, True):
        slots = sorted(a for q in (0, 1) for a in m.kernel_access("put_kc", permuted=permuted, arg0=q))
        assert slots == list(range(0, 2048, 16))
    slots = sorted(a for q in (0, 1) for a in m.kernel_access("put_ks", arg0=q))
    assert slots == list(range(0, 2048, 16))
    slots = sorted(a for q in range(4) for a in m.kernel_access("put_strip", arg0=q))
    assert slots == list(range(0, 4096, 16))
    slots = sorted(a for j in (0, 1) for a in m.kernel_access("put_result", arg0=j))
    assert slots == list(range(0, 2048, 16))
    # fp32 tile: the linear map, the operand map along k and the operand map across k each name every float once
    lib32 = [sorted(a for j in range(4) for a in m.kernel_access("put_f32", arg0=j)),
             sorted(a for q in range(4) for a in m.kernel_access("get_f32_kc", arg0=q)),
             sorted(a for q in range(4) for a in m.kernel_access("get_f32_kc", permuted=True, arg0=q))]
    assert lib32[0] == lib32[1] == lib32[2] and len(set(lib32[0])) == 256
    floats = sorted(a for t in range(16) for a in m.kernel_access("get_f32_ks", arg0=t))
    assert len(set(floats)) == 1024 and set(a - a % 16 for a in floats) == set(lib32[0])
    # operand reads of a [index][k] tile: lane (i, h) finds piece 2 * step + h of the row written for it
    lib = m.index_lib()
    for permuted in (False, True):
        where = {}
        for q in (0, 1):
            for lane, a in enumerate(m.kernel_access("put_kc", permuted=permuted, arg0=q)):
                c = lane + 64 * q
                where[a] = (c >> 2, c & 3)           # (global row, piece)
        for step in (0, 1):
            for lane, a in enumerate(m.kernel_access("get_kc", arg0=step)):
                row, piece = where[a]
                want = lib.bsa_perm16(lane & 31) if permuted else lane & 31
                assert (row, piece) == (want, 2 * step + (lane >> 5))


def test_perm16_is_a_permutation_with_the_accumulator_property():
    lib = m.index_lib()
    perm = [lib.bsa_perm16(i) for i in range(32)]
    assert sorted(perm) == list(range(32))
    assert [lib.bsa_invperm16(perm[i]) for i in range(32)] == list(range(32))
    # accumulator register v of lane half h holds MFMA row 8 * (v / 4) + 4 * h + v % 4: after the
    # permutation that is logical index 16 * h + v
    for h in (0, 1):
        for v in range(16):
            assert perm[8 * (v // 4) + 4 * h + v % 4] == 16 * h + v
