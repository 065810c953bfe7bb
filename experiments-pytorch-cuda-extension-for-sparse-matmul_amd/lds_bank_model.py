"""Bank model of the CDNA4 (gfx950) LDS for checking tile layouts.

Counterpart of the reference's ``bank_conflict_simulator.py`` (lines 17-30 and
46-71: 32 banks of 4 bytes, 32-lane warps, a per-thread index function replayed
into the set of banks each warp touches).  The machine modelled here is
different:

* banks are 4 bytes wide; a wavefront has 64 lanes; an access of ``width`` bytes
  per lane is served in phases of ``banks * 4 / width`` consecutive lanes;
* inside a phase, different dwords that fall into the same bank are served one
  after the other; lanes reading the same dword share one access (broadcast).

The geometry (64 banks, 256 bytes per clock: 64 lanes per phase for b32, 32 for
b64 and the transposing ``ds_read_b64_tr_b16``, 16 for b128) is what the timing
probe ``csrc/lds_bank_probe.hip`` shows on the MI355X: 16 lanes of a b128 read
at stride 64 / 128 / 256 bytes cost 4 / 8 / 16 clocks for their phase, any
permutation of 16 lanes inside one 256-byte window is free, and a pattern that
uses only banks 0-31 runs at half rate (which rules out a 32-bank LDS).  The
model is necessary, not sufficient: two read patterns that it calls free ran at
half rate on the hardware (one 16-byte piece of 32 rows of 64 bytes, with a
different piece permutation in lanes 16-31 than in lanes 0-15), so every access
map the kernels use is also timed on the hardware with ``--probe``.

    python lds_bank_model.py                          # model verdict for the tile layouts in use
    python lds_bank_model.py --probe ./lds_bank_probe  # and the clocks the hardware takes (on a GPU box)
"""
import ctypes
import os
from typing import List, Sequence

MODELS = {"banks64": 64}
BANK_BYTES = 4
WAVE = 64


def phases(width: int, banks: int = 64) -> List[range]:
    """Lane groups served together for an access of ``width`` bytes per lane."""
    lanes = max(1, min(WAVE, banks * BANK_BYTES // width))
    return [range(s, s + lanes) for s in range(0, WAVE, lanes)]


def phase_cost(addresses: Sequence[int], width: int, lanes: range, banks: int = 64) -> int:
    """Clocks one phase takes: the largest number of distinct dwords in one bank."""
    per_bank = {}
    for lane in lanes:
        for dword in range(addresses[lane] // BANK_BYTES, (addresses[lane] + width + BANK_BYTES - 1) // BANK_BYTES):
            per_bank.setdefault(dword % banks, set()).add(dword)
    return max((len(v) for v in per_bank.values()), default=0)


def access_cost(addresses: Sequence[int], width: int, banks: int = 64) -> int:
    """Clocks a 64-lane access takes; the conflict-free figure is ``ideal_cost(width, banks)``."""
    assert len(addresses) == WAVE
    assert all(a % min(width, 16) == 0 for a in addresses), "misaligned LDS access"
    return sum(phase_cost(addresses, width, p, banks) for p in phases(width, banks))


def ideal_cost(width: int, banks: int = 64) -> int:
    return WAVE * width // (banks * BANK_BYTES)


def conflict_free(addresses: Sequence[int], width: int) -> bool:
    """True when the access is free of conflicts under every bank geometry in MODELS."""
    return all(access_cost(addresses, width, b) == ideal_cost(width, b) for b in MODELS.values())


# ---- the layouts the kernels use, through the host build of their index arithmetic ----------
_LIB = None


def index_lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "liblds_index.so")
        if not os.path.exists(path):
            raise ImportError(f"{path} is missing: run csrc/build.py")
        _LIB = ctypes.CDLL(path)
        _LIB.bsa_lds_access.argtypes = [ctypes.c_char_p] + [ctypes.c_int] * 4 + [ctypes.POINTER(ctypes.c_int)]
    return _LIB


def kernel_access(name: str, permuted: bool = False, arg0: int = 0, arg1: int = 0, arg2: int = 0) -> List[int]:
    """Per-lane byte addresses of one LDS access of the kernels (see csrc/lds_index_math.hpp)."""
    buf = (ctypes.c_int * WAVE)()
    if index_lib().bsa_lds_access(name.encode(), int(permuted), arg0, arg1, arg2, buf) != 0:
        raise KeyError(name)
    return list(buf)


# (name, bytes per lane, argument sets): every LDS access the matmul kernels make
KERNEL_ACCESSES = [
    ("put_kc", 16, [dict(permuted=p, arg0=q) for p in (False, True) for q in (0, 1)]),
    ("get_kc", 16, [dict(arg0=s) for s in (0, 1)]),
    ("put_ks", 16, [dict(arg0=q) for q in (0, 1)]),
    ("get_ks", 8, [dict(permuted=p, arg0=s, arg1=h) for p in (False, True) for s in (0, 1) for h in (0, 1)]),
    ("put_strip", 16, [dict(arg0=q) for q in range(4)]),
    ("put_strip_swapped", 16, [dict(arg0=q) for q in range(4)]),
    ("get_kc_tr_swapped", 8, [dict(arg0=s, arg1=h) for s in (0, 1) for h in (0, 1)]),
    ("get_strip", 8, [dict(permuted=p, arg0=s + 2 * h, arg1=x0)
                      for p in (False, True) for s in (0, 1) for h in (0, 1) for x0 in (0, 32)]),
    ("put_strip16", 16, [dict(arg0=q) for q in range(4)]),
    ("get_strip16", 8, [dict(arg0=t, arg1=h) for t in range(4) for h in (0, 1)]),
    ("put_result", 16, [dict(arg0=j) for j in (0, 1)]),
    ("get_linear", 16, [dict(arg0=q) for q in (0, 1)]),
    # fp32 tiles: written and read back linearly (put_f32: both directions), read as MFMA operands along k
    # (get_f32_kc: also the write of the SDD result) and across k (get_f32_ks)
    ("put_f32", 16, [dict(arg0=j) for j in range(4)]),
    ("get_f32_kc", 16, [dict(permuted=p, arg0=q) for p in (False, True) for q in range(4)]),
    ("get_f32_ks", 4, [dict(permuted=p, arg0=t) for p in (False, True) for t in range(16)]),
]


# Accesses that are NOT conflict-free by design, with the clocks the model must find over the ideal: the linear
# access of an fp32 tile takes the 8 pieces of two neighbouring rows per phase, whose windows share 4 of the 64
# banks (csrc/lds_index_math.hpp says why that mapping is kept).
KNOWN_COST_FACTOR = {"put_f32": 2}

# how the probe binary (csrc/lds_bank_probe.hip) issues each access
PROBE_OPS = {"put_kc": "w128", "put_ks": "w128", "put_strip": "w128", "put_strip_swapped": "w128", "put_result": "w128", "put_strip16": "w128", "get_strip16": "tr64",
             "get_kc": "b128", "get_linear": "b128", "put_f32": "w128", "get_f32_kc": "b128", "get_f32_ks": "b32", "get_ks": "tr64", "get_strip": "tr64", "get_kc_tr_swapped": "tr64"}


def _probe(binary: str, op: str, addresses: Sequence[int]) -> float:
    import subprocess
    out = subprocess.run([binary, op, ",".join(str(a) for a in addresses), "x"], capture_output=True, text=True,
                         check=True).stdout
    return float(out.split()[-1])


if __name__ == "__main__":
    import sys
    probe = sys.argv[sys.argv.index("--probe") + 1] if "--probe" in sys.argv else None
    linear = {}
    if probe:
        for op, step in (("b128", 16), ("w128", 16), ("tr64", 8)):
            linear[op] = _probe(probe, op, [step * lane for lane in range(WAVE)])
            print(f"linear      {op:5s} measured {linear[op]:.2f} ticks per wave-instruction (conflict-free yardstick)")
    for name, width, variants in KERNEL_ACCESSES:
        costs = {m: sorted({access_cost(kernel_access(name, **kw), width, b) for kw in variants})
                 for m, b in MODELS.items()}
        ideal = {m: ideal_cost(width, b) for m, b in MODELS.items()}
        line = f"{name:11s} b{8 * width:<4d} {len(variants):2d} variants  model clocks {costs}  ideal {ideal}"
        if probe:
            op = PROBE_OPS[name]
            got = [_probe(probe, op, kernel_access(name, **kw)) for kw in variants]
            line += f"  measured {min(got):.2f}..{max(got):.2f} (linear {linear[op]:.2f})"
        print(line)
