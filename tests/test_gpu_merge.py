"""CrossMerge fused into the kernels (merge = 1): the forward adds weight * result of every group channel
into one fp32 channel per feature, the backward reads the merged gradient and returns
weight * d(weight).  Checked against the two-step construction the fused path replaces: the same kernels
with merge = 0 (themselves pinned against the float64 oracle in the other test files) followed by the
weighted sum over the groups, and its autograd."""
import numpy as np
import pytest
import torch

import capi
from oracle import snd_oracle as O
from oracle import snd_oracle_c as OC
from test_gpu_corners import flip_groups_np
from test_gpu_fwd import relerr

pytestmark = pytest.mark.gpu


def _case(gpu_device, Bt, Dm, H, W, N, K, dtype, seed, shared_u):
    d = O.make_inputs(Bt, Dm, H, W, N=N, K=K, seed=seed)
    t = {k: torch.from_numpy(v).to(gpu_device) for k, v in d.items()}
    for k in ("u", "delta", "B", "C"):
        t[k] = t[k].to(dtype)
    rg = Dm // K
    if shared_u:
        t["u"] = t["u"][:, :rg].contiguous()
    g = torch.Generator(device=gpu_device)
    g.manual_seed(seed)
    t["w"] = (0.5 + torch.rand(Dm, device=gpu_device, generator=g)) * torch.where(torch.rand(Dm, device=gpu_device, generator=g) < 0.3, -1.0, 1.0)
    t["dout_m"] = torch.randn(Bt, rg, H, W, device=gpu_device, generator=g)
    return t, rg


# fp32 inputs: both paths run the same arithmetic per channel; only the order of the sums over the groups
# (float atomics) and of the accumulated gradients differs, hence 1e-5 and not bit equality.
@pytest.mark.parametrize("Bt,Dm,H,W,N,K,dtype,sched,dirs,shared_u,weighted", [
    (2, 32, 19, 27, 16, 4, torch.float32, capi.SCHED_PLANE, capi.DIR_CORNERS, True, True),
    (2, 32, 19, 27, 16, 4, torch.float32, capi.SCHED_STRIPS, capi.DIR_CORNERS, False, True),
    (1, 64, 56, 56, 16, 4, torch.float32, capi.SCHED_AUTO, capi.DIR_CORNERS, True, False),     # wide planes: gathered out rows
    (1, 24, 9, 33, 8, 4, torch.float32, capi.SCHED_PLANE, capi.DIR_TOPLEFT, False, True),     # 8-state kernels, top-left only
    (1, 40, 14, 14, 16, 4, torch.bfloat16, capi.SCHED_AUTO, capi.DIR_CORNERS, True, True),      # 7x7 tiles, direct stores, partial chunk
    (2, 8, 33, 70, 1, 4, torch.float32, capi.SCHED_AUTO, capi.DIR_CORNERS, True, True),        # row-segment kernels, two segments
    (1, 8, 20, 64, 2, 4, torch.bfloat16, capi.SCHED_AUTO, capi.DIR_CORNERS, False, True),
    (1, 8, 12, 600, 1, 4, torch.bfloat16, capi.SCHED_AUTO, capi.DIR_CORNERS, True, True),      # two columns per lane
    (1, 12, 17, 40, 3, 2, torch.float32, capi.SCHED_AUTO, capi.DIR_CORNERS, True, False),      # two groups, three states
    (2, 24, 14, 14, 1, 4, torch.float32, capi.SCHED_WAVEFRONT, capi.DIR_CORNERS, True, True),  # four planes per wave, 6 channels per group
    (2, 28, 9, 30, 2, 4, torch.bfloat16, capi.SCHED_WAVEFRONT, capi.DIR_CORNERS, False, True), # two planes per wave, 7 channels per group
    (2, 40, 7, 7, 1, 4, torch.float32, capi.SCHED_WAVEFRONT, capi.DIR_CORNERS, True, True),    # eight planes per wave, 10 channels per group
    (1, 8, 9, 1100, 2, 4, torch.float32, capi.SCHED_AUTO, capi.DIR_CORNERS, True, True),       # a wide plane: three column groups
    (1, 8, 6, 700, 1, 4, torch.bfloat16, capi.SCHED_WAVEFRONT, capi.DIR_CORNERS, False, True), # odd-free width 700 > 512 with one state: two columns per lane, six segments
    (1, 8, 6, 701, 1, 4, torch.float32, capi.SCHED_WAVEFRONT, capi.DIR_CORNERS, True, False),  # odd width: one column per lane, eleven segments in two groups
])
def test_fused_merge_matches_two_steps(gpu_device, Bt, Dm, H, W, N, K, dtype, sched, dirs, shared_u, weighted):
    print("merge", Bt, Dm, H, W, N, K, dtype, sched, dirs, shared_u, weighted, flush=True)
    t, rg = _case(gpu_device, Bt, Dm, H, W, N, K, dtype, 5, shared_u)
    w = t["w"] if weighted else None
    wv = t["w"] if weighted else torch.ones(Dm, device=gpu_device)
    args = (t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"])
    # two steps: every channel's result, then the weighted sum over the groups
    f0 = capi.FwdCall(*args, True, True, None, True, sched, dirs)
    f0.launch()
    want = (f0.out.view(Bt, K, rg, H, W) * wv.view(1, K, rg, 1, 1)).sum(1)
    f1 = capi.FwdCall(*args, True, True, None, True, sched, dirs, True, w)
    f1.launch()
    f1.launch()                                   # the call clears the merged output itself: no doubling
    torch.cuda.synchronize()
    assert tuple(f1.out.shape) == (Bt, rg, H, W)
    assert relerr(f1.out.cpu().numpy(), want.cpu().numpy()) <= 1e-5
    # backward: the merged gradient against its weighted broadcast fed to the unfused kernel
    dout_full = (t["dout_m"].unsqueeze(1) * wv.view(1, K, rg, 1, 1)).reshape(Bt, Dm, H, W).contiguous()
    b0 = capi.BwdCall(*args, dout_full, f0.x, f0.x_v, True, None, f0.x_sd, sched, dirs)
    b0.launch()
    b1 = capi.BwdCall(*args, t["dout_m"], f1.x, f1.x_v, True, None, f1.x_sd, sched, dirs, True, w)
    b1.launch()
    torch.cuda.synchronize()
    tol = 1e-5 if dtype == torch.float32 else 1e-2     # du / ddelta are rounded to the 16-bit input dtype
    for nm in ("du", "ddelta", "dA", "dB", "dC", "dD", "dbias"):
        a, r = getattr(b1, nm).float().cpu().numpy(), getattr(b0, nm).float().cpu().numpy()
        assert relerr(a, r) <= tol, (nm, relerr(a, r))
    # weight * d(weight) per channel = weight * <merged dout, result of the channel>
    want_w = wv * (f0.out.view(Bt, K, rg, H, W) * t["dout_m"].unsqueeze(1)).sum((0, 3, 4)).reshape(-1)
    assert relerr(b1.dmerge.cpu().numpy(), want_w.cpu().numpy()) <= (1e-4 if dtype == torch.float32 else 1e-2)


def test_fused_merge_against_oracle(gpu_device):
    """The merged output and its gradients against the float64 oracle through flipped copies, fp32, 1e-4."""
    Bt, Dm, H, W, N, K = 1, 16, 21, 30, 16, 4
    d = O.make_inputs(Bt, Dm, H, W, N=N, K=K, seed=9)
    rg = Dm // K
    rng = np.random.default_rng(9)
    w = rng.uniform(0.5, 1.5, Dm).astype(np.float32)
    dout_m = rng.standard_normal((Bt, rg, H, W)).astype(np.float32)
    t = {k: torch.from_numpy(v).to(gpu_device) for k, v in d.items()}
    tw, tdo = torch.from_numpy(w).to(gpu_device), torch.from_numpy(dout_m).to(gpu_device)
    args = (t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"])
    f = capi.FwdCall(*args, True, True, None, True, capi.SCHED_AUTO, capi.DIR_CORNERS, True, tw)
    f.launch()
    b = capi.BwdCall(*args, tdo, f.x, f.x_v, True, None, f.x_sd, capi.SCHED_AUTO, capi.DIR_CORNERS, True, tw)
    b.launch()
    torch.cuda.synchronize()
    fu, fd, fB, fC = (flip_groups_np(d[k], K) for k in ("u", "delta", "B", "C"))
    out_g = flip_groups_np(OC.fwd(fu, fd, d["A"], fB, fC, d["D"], d["delta_bias"], True, None, real="f64"), K)
    ref = (out_g.reshape(Bt, K, rg, H, W) * w.reshape(1, K, rg, 1, 1)).sum(1)
    assert relerr(f.out.cpu().numpy(), ref) <= 1e-4
    dout_full = (dout_m[:, None] * w.reshape(1, K, rg, 1, 1)).reshape(Bt, Dm, H, W)
    g = OC.bwd(fu, fd, d["A"], fB, fC, d["D"], d["delta_bias"], flip_groups_np(np.ascontiguousarray(dout_full), K), True, None, real="f64")
    gref = [flip_groups_np(g[0], K), flip_groups_np(g[1], K), g[2], flip_groups_np(g[3], K), flip_groups_np(g[4], K), g[5], g[6]]
    for nm, a, r in zip(["du", "ddelta", "dA", "dB", "dC", "dD", "ddelta_bias"], [b.du, b.ddelta, b.dA, b.dB, b.dC, b.dD, b.dbias], gref):
        assert relerr(a.cpu().numpy(), r) <= 1e-4, (nm, relerr(a.cpu().numpy(), r))
    ref_w = w * (out_g.reshape(Bt, K, rg, H, W) * dout_m[:, None]).sum((0, 3, 4)).reshape(-1)
    assert relerr(b.dmerge.cpu().numpy(), ref_w) <= 1e-4


@pytest.mark.parametrize("wshape", [None, (4,), (4, 1), (4, 6)])
@pytest.mark.parametrize("N", [16, 1])
def test_cross_scan_2d_fused_autograd(gpu_device, wshape, N):
    """cross_scan_2d (one kernel call each way) against scan + cross_merge, all gradients including the
    merge weights; one weight is exactly zero (its gradient does not vanish)."""
    import selective_nd_scan as snd
    from selective_nd_scan.cross_scan import cross_scan_2d_unfused
    torch.manual_seed(11)
    Bt, Cf, H, W, K = 2, 6, 18, 23, 4
    dev = gpu_device
    x = torch.randn(Bt, Cf, H, W, device=dev)
    delta = 0.1 * torch.randn(Bt, K * Cf, H, W, device=dev)
    A = -torch.rand(K * Cf, N, device=dev) - 0.2
    Bm, Cm = torch.randn(Bt, K, N, H, W, device=dev), torch.randn(Bt, K, N, H, W, device=dev)
    D, bias = torch.randn(K * Cf, device=dev), 0.1 * torch.randn(K * Cf, device=dev)
    wt = None
    if wshape is not None:
        wt = torch.rand(*wshape, device=dev) + 0.5
        wt.view(-1)[1] = 0.0
    leaves = [x, delta, A, Bm, Cm, D, bias] + ([wt] if wt is not None else [])
    res = []
    for fn in (snd.cross_scan_2d, cross_scan_2d_unfused):
        ls = [v.clone().requires_grad_(True) for v in leaves]
        y = fn(ls[0], ls[1], ls[2], ls[3], ls[4], ls[5], ls[6], True, ls[7] if wt is not None else None)
        go = torch.randn(y.shape, device=dev, generator=torch.Generator(device=dev).manual_seed(1))
        y.backward(go)
        res.append([y.detach()] + [v.grad for v in ls])
    names = ["out", "dx", "ddelta", "dA", "dB", "dC", "dD", "dbias", "dw"]
    for nm, a, r in zip(names, res[0], res[1]):
        assert a.shape == r.shape, nm
        assert relerr(a.cpu().numpy(), r.cpu().numpy()) <= 1e-4, (nm, relerr(a.cpu().numpy(), r.cpu().numpy()))


def test_merge_argument_checks(gpu_device):
    d = O.make_inputs(1, 8, 9, 10, N=4, K=4, seed=1)
    t = {k: torch.from_numpy(v).to(gpu_device) for k, v in d.items()}
    args = (t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"])
    f = capi.FwdCall(*args, True, True, None, True, capi.SCHED_AUTO, capi.DIR_CORNERS, True, None)
    f.params.out_dtype = capi.SND_BF16              # merged output must be fp32
    assert capi.lib().snd_fwd(capi.C.byref(f.params), torch.cuda.current_stream().cuda_stream) != 0
    f.params.out_dtype, f.params.merge = capi.SND_F32, 2
    assert capi.lib().snd_fwd(capi.C.byref(f.params), torch.cuda.current_stream().cuda_stream) != 0
    import selective_nd_scan as snd
    with pytest.raises(ValueError):
        snd.selective_nd_scan_merged(*args, True, None, 1, torch.ones(3, device=gpu_device))
    with pytest.raises(RuntimeError):
        snd.fwd(*args, True, False, None, 1, -1, True, None)      # out_float=False with merge
