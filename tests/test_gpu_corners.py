"""Per-group scan origin (directions = 1): group g starts at corner g % 4 inside the kernels.
Pinned by flip equivalence: the result must equal flipping that group's inputs, scanning from the
top-left corner (the oracle, which follows the reference), and flipping the per-pixel results back."""
import numpy as np
import pytest
import torch

import capi
from oracle import snd_oracle as O
from oracle import snd_oracle_c as OC
from test_gpu_fwd import relerr

pytestmark = pytest.mark.gpu
FLIPS = ((False, False), (False, True), (True, False), (True, True))


def flip_np(a, k):
    fv, fh = FLIPS[k % 4]
    if fv:
        a = a[..., ::-1, :]
    if fh:
        a = a[..., ::-1]
    return a


def flip_groups_np(a, G):
    """[B, G*r, H, W] or [B, G, N, H, W]: group g to / from the orientation of corner g % 4."""
    if a.ndim == 5:
        return np.ascontiguousarray(np.stack([flip_np(a[:, g], g) for g in range(G)], 1))
    Bt, Dm, H, W = a.shape
    v = a.reshape(Bt, G, Dm // G, H, W)
    return np.ascontiguousarray(np.stack([flip_np(v[:, g], g) for g in range(G)], 1).reshape(Bt, Dm, H, W))


@pytest.mark.parametrize("Bt,Dm,H,W,N,K,sched", [
    (2, 16, 19, 27, 16, 4, capi.SCHED_PLANE),
    (2, 16, 19, 27, 16, 4, capi.SCHED_STRIPS),
    (1, 64, 56, 56, 16, 4, capi.SCHED_AUTO),
    (1, 24, 9, 33, 4, 8, capi.SCHED_PLANE),      # 8 groups: corners repeat with period 4; 8-state kernels
    (1, 8, 40, 12, 16, 2, capi.SCHED_STRIPS),    # 2 groups: corners 0 and 1 only
])
def test_corner_directions_match_flipped_oracle(gpu_device, Bt, Dm, H, W, N, K, sched):
    print("corners", Bt, Dm, H, W, N, K, sched, flush=True)
    d = O.make_inputs(Bt, Dm, H, W, N=N, K=K, seed=21)
    t = {k: torch.from_numpy(v).to(gpu_device) for k, v in d.items()}
    args = (t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"])
    f = capi.FwdCall(*args, True, True, None, True, sched, capi.DIR_CORNERS)
    f.launch()
    b = capi.BwdCall(*args, t["dout"], f.x, f.x_v, True, None, f.x_sd, sched, capi.DIR_CORNERS)
    b.launch()
    torch.cuda.synchronize()
    fu, fd, fB, fC, fdo = (flip_groups_np(d[k], K) for k in ("u", "delta", "B", "C", "dout"))
    ref = flip_groups_np(OC.fwd(fu, fd, d["A"], fB, fC, d["D"], d["delta_bias"], True, None, real="f64"), K)
    g = OC.bwd(fu, fd, d["A"], fB, fC, d["D"], d["delta_bias"], fdo, True, None, real="f64")
    gref = [flip_groups_np(g[0], K), flip_groups_np(g[1], K), g[2], flip_groups_np(g[3], K), flip_groups_np(g[4], K), g[5], g[6]]
    assert relerr(f.out.cpu().numpy(), ref) <= 1e-4
    for nm, a, r in zip(["du", "ddelta", "dA", "dB", "dC", "dD", "ddelta_bias"],
                        [b.du, b.ddelta, b.dA, b.dB, b.dC, b.dD, b.dbias], gref):
        assert relerr(a.cpu().numpy(), r) <= 1e-4, (nm, relerr(a.cpu().numpy(), r))
    # and it is not the top-left result
    f0 = capi.FwdCall(*args, True, True, None, False, sched, capi.DIR_TOPLEFT)
    f0.launch()
    torch.cuda.synchronize()
    assert relerr(f0.out.cpu().numpy(), ref) > 1e-3


def test_four_corner_block_in_kernel_equals_flipped_copies(gpu_device):
    """Autograd level: directions=1 against the flip / scan / un-flip construction, bf16 inputs."""
    import selective_nd_scan as snd
    torch.manual_seed(3)
    Bt, Cf, H, W, N = 2, 8, 21, 14, 16
    dev = gpu_device
    x = torch.randn(Bt, Cf, H, W, device=dev).bfloat16().requires_grad_()
    delta = (0.1 * torch.randn(Bt, 4 * Cf, H, W, device=dev)).bfloat16().requires_grad_()
    A = (-torch.rand(4 * Cf, N, device=dev) * 4 - 0.1).requires_grad_()
    Bm = torch.randn(Bt, 4, N, H, W, device=dev).bfloat16().requires_grad_()
    Cm = torch.randn(Bt, 4, N, H, W, device=dev).bfloat16().requires_grad_()
    D = torch.randn(4 * Cf, device=dev).requires_grad_()
    bias = torch.randn(4 * Cf, device=dev).requires_grad_()
    w = torch.rand(4, Cf, device=dev).requires_grad_()
    leaves = (x, delta, A, Bm, Cm, D, bias, w)

    y1 = snd.cross_scan_2d(x, delta, A, Bm, Cm, D, bias, True, w)
    g1 = torch.autograd.grad(y1.square().sum(), leaves)
    y2 = snd.cross_merge(snd.four_corner_scan_by_flips(snd.cross_scan(x), delta, A, Bm, Cm, D, bias, True, True), w)
    g2 = torch.autograd.grad(y2.square().sum(), leaves)
    assert y1.shape == (Bt, Cf, H, W) and y1.dtype == torch.float32
    assert relerr(y1.detach().cpu().numpy(), y2.detach().cpu().numpy()) <= 1e-5
    for a, b_ in zip(g1, g2):
        assert relerr(a.float().cpu().numpy(), b_.float().cpu().numpy()) <= 2e-2, relerr(a.float().cpu().numpy(), b_.float().cpu().numpy())


@pytest.mark.parametrize("dirs", [capi.DIR_TOPLEFT, capi.DIR_CORNERS])
def test_u_shared_by_the_groups_equals_repeated_u(gpu_device, dirs):
    """u with dim / n_groups channels (one feature map scanned by every group) against the same
    call on u repeated per group: identical out and gradients, du summed over the groups."""
    Bt, r, H, W, N, K = 2, 12, 23, 18, 16, 4
    d = O.make_inputs(Bt, K * r, H, W, N=N, K=K, seed=31)
    t = {k: torch.from_numpy(v).to(gpu_device) for k, v in d.items()}
    x = t["u"][:, :r].contiguous()
    rest = (t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"])
    res = []
    for u in (x, x.repeat(1, K, 1, 1)):
        f = capi.FwdCall(u, *rest, True, True, None, True, capi.SCHED_AUTO, dirs)
        f.launch()
        g = capi.bwd(u, *rest, t["dout"], f.x, f.x_v, True, None, f.x_sd, None, capi.SCHED_AUTO, dirs)
        torch.cuda.synchronize()
        res.append((f.out, g))
    (out_s, g_s), (out_r, g_r) = res
    assert out_s.shape == (Bt, K * r, H, W) and torch.equal(out_s, out_r)
    assert g_s[0].shape == x.shape
    assert relerr(g_s[0].cpu().numpy(), g_r[0].view(Bt, K, r, H, W).sum(1).cpu().numpy()) <= 1e-6
    assert torch.equal(g_s[1], g_r[1])
    for a, b_ in zip(g_s[2:7], g_r[2:7]):
        assert relerr(a.cpu().numpy(), b_.cpu().numpy()) <= 1e-5      # atomic sums: order may differ
