"""Writes the golden fixtures of this directory from the pinned CPU oracle.

    python tests/golden/make_golden.py

The reference holds no golden vectors for the scan, so these are produced by the fp64 C
oracle (oracle/m2d_oracle.c), itself pinned by tests/test_oracle.py.  Inputs are stored
as drawn (fp32); outputs and the nine gradients are fp64.

  cfg0_B2_E32_14x14_N16.npz   the reference-CPU-runnable benchmark case
  ragged_B3_E4_5x9_N16.npz    non-square, batch not a multiple of anything
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import scan_oracle as so  # noqa: E402

CASES = {
    "cfg0_B2_E32_14x14_N16": dict(B=2, H=14, W=14, E=32, N=16, seed=1234),
    "ragged_B3_E4_5x9_N16": dict(B=3, H=5, W=9, E=4, N=16, seed=99),
}


def main():
    cs = so.CScan()
    here = os.path.dirname(os.path.abspath(__file__))
    for name, kw in CASES.items():
        inp = so.make_inputs(**kw)
        a = [inp[k] for k in so.INPUT_NAMES]
        y = cs.forward(*a)
        g = cs.backward(*a, inp["dy"])
        blob = {"in_" + k: v.numpy() for k, v in inp.items()}
        blob["y"] = y
        blob.update(g)
        blob["meta"] = np.array([kw[k] for k in ("B", "H", "W", "E", "N", "seed")], dtype=np.int64)
        np.savez_compressed(os.path.join(here, name + ".npz"), **blob)
        print(name, {k: v.shape for k, v in blob.items() if k != "meta"})


if __name__ == "__main__":
    main()
