"""Parity at the plane sizes of the benchmark configurations (channel/batch counts reduced so the
C oracle finishes in seconds): long planes exercise the strip-to-strip and tile-to-tile carries over
hundreds of tiles, non-square / non-multiple-of-8 extents, bf16 inputs with fp32 state, and N = 1."""
import numpy as np
import pytest
import torch

import capi
from oracle import snd_oracle as O
from oracle import snd_oracle_c as OC
from test_gpu_fwd import relerr

pytestmark = pytest.mark.gpu
NAMES = ["du", "ddelta", "dA", "dB", "dC", "dD", "ddelta_bias"]

CONFIGS = [
    # name, Bt, Dm, H, W, N, K, dtype
    ("c1-plane", 2, 16, 56, 56, 16, 4, torch.float32),
    ("c2-plane", 3, 64, 14, 14, 16, 4, torch.bfloat16),
    ("c3-plane", 1, 8, 200, 336, 16, 4, torch.float32),
    ("c4-plane", 1, 8, 512, 512, 16, 4, torch.bfloat16),
    ("c4-plane-n1", 1, 8, 512, 512, 1, 4, torch.bfloat16),
    ("odd", 1, 4, 61, 43, 16, 2, torch.float32),
    # planes that are walked in 7x7 tiles (fewer padded cells than with 8x8)
    ("stage-28", 2, 16, 28, 28, 16, 4, torch.float32),
    ("stage-7", 2, 32, 7, 7, 16, 4, torch.bfloat16),
    ("te7-ragged", 1, 8, 20, 33, 8, 2, torch.float32),
    ("te7-row", 3, 4, 6, 40, 16, 1, torch.float16),
]


@pytest.mark.parametrize("name,Bt,Dm,H,W,N,K,dtype", CONFIGS)
def test_config_plane_sizes(gpu_device, name, Bt, Dm, H, W, N, K, dtype):
    print("config", name, flush=True)
    d = O.make_inputs(Bt, Dm, H, W, N=N, K=K, seed=11)
    t = {k: torch.from_numpy(v).to(gpu_device) for k, v in d.items()}
    for k in ("u", "delta", "B", "C"):
        t[k] = t[k].to(dtype)
    out, x, x_v, x_sd = capi.fwd(t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"], True, True, None)
    g = capi.bwd(t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"], t["dout"], x, x_v, True, None, x_sd)
    torch.cuda.synchronize()
    # float64 C oracle on the values the kernel saw (rounded inputs)
    r = {k: t[k].float().cpu().numpy() for k in ("u", "delta", "B", "C")}
    ref = OC.fwd(r["u"], r["delta"], d["A"], r["B"], r["C"], d["D"], d["delta_bias"], True, None, real="f64")
    gref = OC.bwd(r["u"], r["delta"], d["A"], r["B"], r["C"], d["D"], d["delta_bias"], d["dout"], True, None, real="f64")
    assert relerr(out.cpu().numpy(), ref) <= 1e-4
    half = dtype != torch.float32
    for nm, a, b_ in zip(NAMES, g, gref):
        tol = 1e-2 if (half and nm in ("du", "ddelta", "dB", "dC")) else 1e-4
        assert relerr(a.float().cpu().numpy(), b_) <= tol, (nm, relerr(a.float().cpu().numpy(), b_))
    if half:
        # headline tolerance for 16-bit inputs: out and every gradient within 1e-2 of the oracle fed the UN-ROUNDED fp32
        # inputs (max|x - ref| / max|ref| per tensor)
        ref32 = OC.fwd(d["u"], d["delta"], d["A"], d["B"], d["C"], d["D"], d["delta_bias"], True, None, real="f64")
        assert relerr(out.cpu().numpy(), ref32) <= 1e-2
        gref32 = OC.bwd(d["u"], d["delta"], d["A"], d["B"], d["C"], d["D"], d["delta_bias"], d["dout"], True, None, real="f64")
        for nm, a, b_ in zip(NAMES, g, gref32):
            e = relerr(a.float().cpu().numpy(), b_)
            print("  un-rounded", nm, "%.2e" % e, flush=True)
            assert e <= 1e-2, (nm, e)
