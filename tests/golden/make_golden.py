"""Writes tests/golden/snd_golden.npz from the pinned float64 oracle (oracle/snd_oracle.py).

The reference ships no golden vectors for selective_nd_scan, so these are the build's own: seeded
inputs (oracle.make_inputs) and the oracle's outputs/gradients, stored as float32.  Run from the
repo root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import snd_oracle as O  # noqa: E402

CASES = {
    # name: (Bt, Dm, H, W, N, K, Dd, seed)
    "c0": (1, 64, 14, 14, 16, 4, None, 0),          # benchmark config 0, forward only
    "small": (2, 8, 11, 13, 16, 4, None, 7),        # ragged tiles, forward + every gradient
    "groups": (1, 6, 9, 10, 5, 2, 3, 8),            # dstate 5, shared delta groups
}


def main():
    out = {}
    for name, (Bt, Dm, H, W, N, K, Dd, seed) in CASES.items():
        d = O.make_inputs(Bt, Dm, H, W, N=N, K=K, seed=seed, Dd=Dd)
        args = (d["u"], d["delta"], d["A"], d["B"], d["C"], d["D"], d["delta_bias"])
        out[name + "/out"] = O.selective_nd_scan_fwd(*args, True).astype(np.float32)
        out[name + "/shape"] = np.array([Bt, Dm, H, W, N, K, Dd or Dm, seed])
        if name != "c0":
            g = O.selective_nd_scan_bwd(*args, d["dout"], True)
            for k, v in zip(("du", "ddelta", "dA", "dB", "dC", "dD", "ddelta_bias"), g):
                out[name + "/" + k] = v.astype(np.float32)
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "snd_golden.npz"), **out)
    print("wrote", len(out), "arrays")


if __name__ == "__main__":
    main()
