"""The VSS-style block on the HIP op against the same block with the scan replaced by the torch
restatement of the reference recurrence (flip / scan / un-flip for the four corners)."""
import copy

import pytest
import torch

from oracle.snd_torch_ref import selective_nd_scan_torch
from test_gpu_fwd import relerr

pytestmark = pytest.mark.gpu


def torch_four_corner_scan(u, delta, A, B, C, D, delta_bias, delta_softplus, out_float):
    import importlib
    cs = importlib.import_module("selective_nd_scan.cross_scan")
    G = B.shape[1]
    if u.shape[1] != A.shape[0]:
        u = u.repeat(1, G, 1, 1)
    f64 = lambda t: t.double().cpu()
    out = selective_nd_scan_torch(f64(cs.flip_groups(u, G)), f64(cs.flip_groups(delta, G)), f64(A), f64(cs.flip_groups(B, G)),
                                  f64(cs.flip_groups(C, G)), f64(D), f64(delta_bias), delta_softplus)
    return cs.flip_groups(out, G).float().to(u.device)


def test_vss_block_forward_backward(gpu_device):
    import selective_nd_scan as snd
    torch.manual_seed(0)
    blk = snd.VSSBlock(d_model=16, d_state=4, ssm_ratio=1.0, mlp_ratio=2.0).to(gpu_device)
    ref = copy.deepcopy(blk)
    ref.op.scan_fn = torch_four_corner_scan
    x = torch.randn(2, 9, 7, 16, device=gpu_device)
    xa, xb = x.clone().requires_grad_(), x.clone().requires_grad_()
    ya, yb = blk(xa), ref(xb)
    assert ya.shape == x.shape
    assert relerr(ya.detach().cpu().numpy(), yb.detach().cpu().numpy()) <= 1e-4
    ya.square().sum().backward()
    yb.square().sum().backward()
    assert relerr(xa.grad.cpu().numpy(), xb.grad.cpu().numpy()) <= 2e-4
    for (name, pa), (_, pb) in zip(blk.named_parameters(), ref.named_parameters()):
        assert pa.grad is not None, name
        assert relerr(pa.grad.cpu().numpy(), pb.grad.cpu().numpy()) <= 5e-4, (name, relerr(pa.grad.cpu().numpy(), pb.grad.cpu().numpy()))


def test_vss_block_bf16_autocast_runs(gpu_device):
    import selective_nd_scan as snd
    torch.manual_seed(1)
    blk = snd.VSSBlock(d_model=32, d_state=16, ssm_ratio=2.0, mlp_ratio=0.0).to(gpu_device)
    x = torch.randn(1, 20, 12, 32, device=gpu_device, requires_grad=True)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y = blk(x)
    y.float().square().mean().backward()
    assert torch.isfinite(y).all() and torch.isfinite(x.grad).all()
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in blk.parameters())
