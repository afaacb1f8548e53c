"""Forward and backward of one call pair must run the same kernel family (each keeps its own saved-state layout in
tensors of the same shapes).  The autograd functions fix the block mapping in forward(); at the C ABI a backward of
the other family finds the wrong tag in the saved state and returns NaN gradients, never plausible numbers."""
import numpy as np
import pytest
import torch

import capi
from oracle import snd_oracle as O
from oracle import snd_oracle_c as OC
from test_gpu_fwd import relerr

pytestmark = pytest.mark.gpu


def _inputs(dev, Bt=2, Dm=8, H=20, W=40, N=1, K=4, seed=11):
    d = O.make_inputs(Bt, Dm, H, W, N=N, K=K, seed=seed)
    t = {k: torch.from_numpy(v).to(dev) for k, v in d.items()}
    return d, t


@pytest.mark.parametrize("fwd_sched,bwd_sched", [(capi.SCHED_PLANE, capi.SCHED_AUTO), (capi.SCHED_WAVEFRONT, capi.SCHED_PLANE),
                                                 (capi.SCHED_STRIPS, capi.SCHED_WAVEFRONT)])
def test_backward_of_the_other_family_returns_nan(gpu_device, fwd_sched, bwd_sched):
    d, t = _inputs(gpu_device)
    st, plan = capi.make_plan(capi.make_shape(t["u"], t["delta"], t["A"], t["B"]))
    assert st == 0 and plan.auto_schedule == capi.SCHED_WAVEFRONT        # AUTO means the row-segment family here
    args = (t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"])
    f = capi.FwdCall(*args, True, True, None, True, fwd_sched)
    f.launch()
    b = capi.BwdCall(*args, t["dout"], f.x, f.x_v, True, None, f.x_sd, bwd_sched)
    b.launch()
    torch.cuda.synchronize()
    for name, g in (("du", b.du), ("ddelta", b.ddelta), ("dA", b.dA), ("dB", b.dB), ("dC", b.dC), ("dD", b.dD), ("dbias", b.dbias)):
        assert torch.isnan(g).all(), name
    # the same saved state with the forward's own family: the true gradients
    b2 = capi.BwdCall(*args, t["dout"], f.x, f.x_v, True, None, f.x_sd, fwd_sched)
    b2.launch()
    torch.cuda.synchronize()
    o = tuple(d[k] for k in ("u", "delta", "A", "B", "C", "D", "delta_bias"))
    gref = OC.bwd(*o, d["dout"], True, None, real="f64")
    for got, ref in zip((b2.du, b2.ddelta, b2.dA, b2.dB, b2.dC, b2.dD, b2.dbias), gref):
        assert relerr(got.cpu().numpy(), ref) <= 1e-4          # fp32: max|x - ref| / max|ref|


def test_autograd_keeps_the_forward_schedule(gpu_device):
    """A default block mapping changed between a forward and its backward does not reach the backward."""
    import selective_nd_scan as snd
    d, t = _inputs(gpu_device, seed=12)
    grads = []
    try:
        for switch in (False, True):
            leaves = {k: t[k].clone().requires_grad_(True) for k in ("u", "delta", "A", "B", "C", "D", "delta_bias")}
            snd.set_schedule(capi.SCHED_PLANE)
            out = snd.selective_nd_scan(leaves["u"], leaves["delta"], leaves["A"], leaves["B"], leaves["C"], leaves["D"],
                                        leaves["delta_bias"], True, True)
            if switch:
                snd.set_schedule(capi.SCHED_AUTO)             # would pick the other kernel family for this shape
            out.backward(t["dout"])
            grads.append([leaves[k].grad.clone() for k in leaves])
    finally:
        snd.set_schedule(capi.SCHED_AUTO)
    o = tuple(d[k] for k in ("u", "delta", "A", "B", "C", "D", "delta_bias"))
    gref = OC.bwd(*o, d["dout"], True, None, real="f64")
    for a, b, ref in zip(grads[0], grads[1], gref):
        assert torch.equal(a, b) or relerr(a.cpu().numpy(), b.cpu().numpy()) <= 1e-5   # (atomic sums: order may differ)
        assert relerr(b.cpu().numpy(), ref) <= 1e-4
