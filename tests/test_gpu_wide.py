"""Planes wider than 1024 columns (the reference's nChunksX > 1 path, selective_scan_oflex.cpp:249):
many column tiles per strip, the out gather over groups of tiles, hand-over rows at hundreds of tiles."""
import pytest
import torch

import capi
from oracle import snd_oracle as O
from oracle import snd_oracle_c as OC
from test_gpu_fwd import relerr

pytestmark = pytest.mark.gpu
NAMES = ["du", "ddelta", "dA", "dB", "dC", "dD", "ddelta_bias"]


@pytest.mark.parametrize("N,dtype,sched", [(16, torch.float32, capi.SCHED_PLANE), (16, torch.float32, capi.SCHED_STRIPS),
                                           (4, torch.float32, capi.SCHED_AUTO), (16, torch.bfloat16, capi.SCHED_STRIPS),
                                           (1, torch.float32, capi.SCHED_AUTO)])
def test_wide_plane(gpu_device, N, dtype, sched):
    print("wide plane", N, dtype, sched, flush=True)
    Bt, Dm, H, W, K = 1, 8, 9, 1500, 2
    d = O.make_inputs(Bt, Dm, H, W, N=N, K=K, seed=31)
    t = {k: torch.from_numpy(v).to(gpu_device) for k, v in d.items()}
    for k in ("u", "delta", "B", "C"):
        t[k] = t[k].to(dtype)
    args = (t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"])
    f = capi.FwdCall(*args, True, True, None, True, sched)
    f.launch()
    b = capi.BwdCall(*args, t["dout"], f.x, f.x_v, True, None, f.x_sd, sched)
    b.launch()
    torch.cuda.synchronize()
    r = {k: t[k].float().cpu().numpy() for k in ("u", "delta", "B", "C")}
    o = (r["u"], r["delta"], d["A"], r["B"], r["C"], d["D"], d["delta_bias"])
    ref = OC.fwd(*o, True, None, real="f64")
    gref = OC.bwd(*o, d["dout"], True, None, real="f64")
    assert relerr(f.out.cpu().numpy(), ref) <= 1e-4
    half = dtype != torch.float32
    for nm, a, w in zip(NAMES, [b.du, b.ddelta, b.dA, b.dB, b.dC, b.dD, b.dbias], gref):
        tol = 1e-2 if (half and nm in ("du", "ddelta", "dB", "dC")) else 1e-4
        assert relerr(a.float().cpu().numpy(), w) <= tol, (nm, relerr(a.float().cpu().numpy(), w))
