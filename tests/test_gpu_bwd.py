"""GPU parity of the HIP backward against the float64 oracle's hand adjoint, through the C ABI.

fp32 inputs: every gradient within max-rel 1e-4 (rel = max|x - ref| / max|ref| per tensor);
bf16 inputs: within 1e-2 of the fp32 oracle.  The oracle's adjoint is itself pinned against
torch.autograd and finite differences in tests/test_oracle_pins.py.
"""
import numpy as np
import pytest
import torch

import capi
from oracle import snd_oracle as O
from test_gpu_fwd import relerr, to_dev

pytestmark = pytest.mark.gpu

NAMES = ["du", "ddelta", "dA", "dB", "dC", "dD", "ddelta_bias", "dA_decay"]


def run_case(dev, Bt, Dm, H, W, N, K, Dd, seed, dtype=torch.float32, softplus=True, use_D=True, use_bias=True,
             decay=None, dout_dtype=torch.float32):
    d = O.make_inputs(Bt, Dm, H, W, N=N, K=K, seed=seed, Dd=Dd)
    if not softplus:
        d["delta"] = np.abs(d["delta"]) + 0.01
    D = d["D"] * (1.0 + 0.1 * np.arange(Dm, dtype=np.float32)) if use_D else None
    bias = d["delta_bias"] if use_bias else None
    dec = None if decay is None else np.array([decay], np.float32)
    t = to_dev(d, dev, dtype)
    tD = None if D is None else torch.from_numpy(D).to(dev)
    tb = None if bias is None else t["delta_bias"]
    tdec = None if dec is None else torch.from_numpy(dec).to(dev)
    dout = t["dout"].to(dout_dtype)
    out, x, x_v, x_sd = capi.fwd(t["u"], t["delta"], t["A"], t["B"], t["C"], tD, tb, softplus, True, tdec)
    grads = capi.bwd(t["u"], t["delta"], t["A"], t["B"], t["C"], tD, tb, dout, x, x_v, softplus, tdec, x_sd)
    torch.cuda.synchronize()
    # oracle on exactly the values the kernel saw (rounded inputs), float64
    f = lambda k: t[k].float().cpu().numpy()
    ref = O.selective_nd_scan_bwd(f("u"), f("delta"), d["A"], f("B"), f("C"), D, bias, dout.float().cpu().numpy(),
                                  softplus, dec)
    ref_out = O.selective_nd_scan_fwd(f("u"), f("delta"), d["A"], f("B"), f("C"), D, bias, softplus, dec)
    errs = {"out": relerr(out.cpu().numpy(), ref_out)}
    for name, gk, gr in zip(NAMES, grads, ref):
        if gr is None:
            assert gk is None, name
            continue
        assert gk is not None, name
        assert tuple(gk.shape) == tuple(gr.shape), (name, gk.shape, gr.shape)
        errs[name] = relerr(gk.float().cpu().numpy(), gr)
    return errs, grads


CASES = [
    # Bt, Dm, H, W, N, K, Dd
    (1, 64, 14, 14, 16, 4, None),      # config-0 shape
    (2, 8, 8, 8, 16, 2, None),         # exactly one tile
    (1, 4, 1, 37, 16, 1, None),        # single row
    (1, 4, 29, 1, 16, 1, None),        # single column
    (2, 12, 19, 23, 16, 4, None),      # ragged strips/tiles, partial channel chunk (3 per group)
    (1, 40, 17, 9, 16, 2, None),       # 20 channels per group: two chunks, second partial
    (1, 6, 17, 9, 5, 2, 3),            # dstate not a power of two, shared delta groups
    (1, 40, 9, 10, 1, 2, None),        # d_state = 1
    (1, 8, 9, 20, 8, 1, 2),
    (1, 16, 24, 16, 12, 1, None),
]


@pytest.mark.parametrize("Bt,Dm,H,W,N,K,Dd", CASES)
def test_bwd_fp32_matches_oracle(gpu_device, Bt, Dm, H, W, N, K, Dd):
    print("case", Bt, Dm, H, W, N, K, Dd, flush=True)
    errs, grads = run_case(gpu_device, Bt, Dm, H, W, N, K, Dd, seed=H * 131 + W)
    assert grads[0].dtype == torch.float32 and grads[3].dtype == torch.float32
    assert grads[1].shape[1] == (Dd or Dm) and grads[6].shape[0] == (Dd or Dm)
    for k, e in errs.items():
        assert e <= 1e-4, (k, e, errs)


def test_bwd_options_off(gpu_device):
    errs, grads = run_case(gpu_device, 2, 8, 10, 13, 16, 2, None, seed=3, softplus=False, use_D=False, use_bias=False)
    assert grads[5] is None and grads[6] is None and grads[7] is None
    for k, e in errs.items():
        assert e <= 1e-4, (k, e, errs)


def test_bwd_a_decay(gpu_device):
    errs, grads = run_case(gpu_device, 2, 8, 11, 12, 16, 2, None, seed=4, decay=0.9)
    assert grads[7] is not None and grads[7].shape == (1,)
    for k, e in errs.items():
        assert e <= 1e-4, (k, e, errs)


@pytest.mark.parametrize("dtype,dout_dtype", [(torch.bfloat16, torch.float32), (torch.bfloat16, torch.bfloat16),
                                              (torch.float16, torch.float32)])
def test_bwd_half_inputs(gpu_device, dtype, dout_dtype):
    errs, grads = run_case(gpu_device, 2, 16, 14, 14, 16, 4, None, seed=5, dtype=dtype, dout_dtype=dout_dtype)
    assert grads[0].dtype == dtype and grads[1].dtype == dtype and grads[3].dtype == dtype and grads[4].dtype == dtype
    assert grads[2].dtype == torch.float32
    # the oracle here saw the rounded inputs, so what is left is the rounding of the 16-bit gradients
    tol = 1e-2 if dtype == torch.bfloat16 else 2e-3
    for k, e in errs.items():
        assert e <= (tol if k in ("du", "ddelta", "dB", "dC") else 1e-4), (k, e, errs)


def test_bwd_twice_over_same_saved_state(gpu_device):
    """The saved state is read-only for bwd, so a second backward gives the same gradients."""
    d = O.make_inputs(1, 8, 19, 21, N=16, K=2, seed=9)
    t = to_dev(d, gpu_device)
    out, x, x_v, x_sd = capi.fwd(t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"], True, True, None)
    g1 = capi.bwd(t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"], t["dout"], x, x_v, True, None, x_sd)
    g2 = capi.bwd(t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"], t["dout"], x, x_v, True, None, x_sd)
    for a, b_, name in zip(g1, g2, NAMES):
        if a is None:
            continue
        assert relerr(b_.cpu().numpy(), a.cpu().numpy()) <= 1e-6, name


def test_bwd_linearity_in_dout_at_scale(gpu_device):
    """Full-size property: every gradient is linear in dout (checked at the stage-1 plane size)."""
    torch.manual_seed(1)
    Bt, Dm, H, W, N, K = 4, 96, 56, 56, 16, 4
    dev = gpu_device
    u = torch.randn(Bt, Dm, H, W, device=dev)
    delta = 0.1 * torch.randn(Bt, Dm, H, W, device=dev)
    bias = torch.log(torch.expm1(torch.exp(torch.empty(Dm, device=dev).uniform_(np.log(1e-3), np.log(1e-1)))))
    A = -torch.arange(1, N + 1, device=dev, dtype=torch.float32).repeat(Dm, 1)
    B = torch.randn(Bt, K, N, H, W, device=dev)
    Cc = torch.randn(Bt, K, N, H, W, device=dev)
    D = torch.ones(Dm, device=dev)
    d1 = torch.randn(Bt, Dm, H, W, device=dev)
    d2 = torch.randn(Bt, Dm, H, W, device=dev)
    out, x, x_v, x_sd = capi.fwd(u, delta, A, B, Cc, D, bias, True, True, None)
    bw = lambda dd: capi.bwd(u, delta, A, B, Cc, D, bias, dd, x, x_v, True, None, x_sd)
    g1, g2, g12 = bw(d1), bw(d2), bw(2.0 * d1 - 3.0 * d2)
    for a, b_, c_, name in zip(g1, g2, g12, NAMES):
        if a is None:
            continue
        assert relerr(c_.cpu().numpy(), (2.0 * a - 3.0 * b_).cpu().numpy()) <= 1e-4, name
