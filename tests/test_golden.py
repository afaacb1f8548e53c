"""Committed golden vectors (tests/golden/snd_golden.npz, written by tests/golden/make_golden.py from the
pinned oracle): the oracle must keep reproducing them (CPU), and the HIP path must match them (GPU)."""
import os

import numpy as np
import pytest

from oracle import snd_oracle as O

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "snd_golden.npz"))
CASES = sorted({k.split("/")[0] for k in G.files})
GRADS = ("du", "ddelta", "dA", "dB", "dC", "dD", "ddelta_bias")


def inputs(name):
    Bt, Dm, H, W, N, K, Dd, seed = (int(v) for v in G[name + "/shape"])
    return O.make_inputs(Bt, Dm, H, W, N=N, K=K, seed=seed, Dd=Dd)


def rel(x, ref):
    return float(np.abs(np.asarray(x, np.float64) - ref).max() / max(np.abs(ref).max(), 1e-30))


@pytest.mark.parametrize("name", CASES)
def test_oracle_reproduces_golden(name):
    d = inputs(name)
    args = (d["u"], d["delta"], d["A"], d["B"], d["C"], d["D"], d["delta_bias"])
    assert rel(O.selective_nd_scan_fwd(*args, True), G[name + "/out"]) <= 1e-6
    if name + "/du" in G.files:
        for k, v in zip(GRADS, O.selective_nd_scan_bwd(*args, d["dout"], True)):
            assert rel(v, G[name + "/" + k]) <= 1e-6, k


@pytest.mark.gpu
@pytest.mark.parametrize("name", CASES)
def test_hip_matches_golden(gpu_device, name):
    import torch
    import capi
    d = inputs(name)
    t = {k: torch.from_numpy(v).to(gpu_device) for k, v in d.items()}
    out, x, x_v, x_sd = capi.fwd(t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"], True, True, None)
    assert rel(out.cpu().numpy(), G[name + "/out"]) <= 1e-4
    if name + "/du" in G.files:
        g = capi.bwd(t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"], t["dout"], x, x_v, True, None, x_sd)
        for k, v in zip(GRADS, g):
            assert rel(v.cpu().numpy(), G[name + "/" + k]) <= 1e-4, k
