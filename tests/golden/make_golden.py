"""Writes tests/golden/layout_tables.json: the block tables of the five benchmark masks,
computed by the BRUTE-FORCE builder (double loops over the definition), so that the
vectorised oracle, the C walk and the device builder can all be held against them.
The reference ships no vectors for this path (it has no tests at all), so these
are derived from the table definition, not from running the reference.

    python tests/golden/make_golden.py
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "experiments-pytorch-cuda-extension-for-sparse-matmul_amd"))

from oracle import layout_oracle as lo  # noqa: E402
import workloads as wl  # noqa: E402


def main():
    masks = {
        "config1": wl.config1()["mask"].numpy(),
        "config2": wl.mask_local_window(64, 2).numpy(),
        "config3_4": wl.mask_causal_local_strided(128).numpy(),
        "config5": wl.mask_bigbird(256, wl._gen(5)).numpy(),
    }
    out = {}
    for name, mask in masks.items():
        entry = {"shape": list(mask.shape), "nnz": int(np.count_nonzero(mask)),
                 "mask_rows_hex": ["%x" % int("".join(map(str, row)), 2) for row in mask.tolist()]}
        for tr, key in ((False, "row"), (True, "col")):
            blocks, offs = lo.create_layout_bruteforce(mask, tr)
            w = np.arange(1, len(blocks) + 1, dtype=np.int64)
            entry[key + "_offsets"] = offs.tolist()
            entry[key + "_blocks_sum"] = int(blocks.astype(np.int64).sum())
            entry[key + "_blocks_wsum"] = int((blocks.astype(np.int64) * w % 1000003).sum())
            entry[key + "_blocks_head"] = blocks[:16].tolist()
        out[name] = entry
    with open(os.path.join(HERE, "layout_tables.json"), "w") as f:
        json.dump(out, f, indent=1)
    print({k: v["nnz"] for k, v in out.items()})


if __name__ == "__main__":
    main()
