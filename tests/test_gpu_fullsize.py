"""The benchmark configurations at their full sizes, with the schedule the library picks by itself
(two bands per plane in c1's backward, pipelined strips in c3 / c4).  The float64 C oracle runs on
one slice that is independent of the rest - one batch image, and for the largest planes one channel
group of it - and the whole result is compared with the whole-plane schedule: everything that is
not an atomic sum must be bit-identical, the atomic sums equal up to summation order."""
import numpy as np
import pytest
import torch

import capi
from oracle import snd_oracle_c as OC
from test_gpu_fwd import relerr

pytestmark = pytest.mark.gpu

FULL = [
    # name, Bt, Dm, H, W, N, K, dtype, oracle batch image, oracle groups, forward AUTO, backward jobs per plane
    ("c1", 64, 192, 56, 56, 16, 4, torch.float32, 37, 4, capi.SCHED_PLANE, 2),
    ("c2", 64, 768, 14, 14, 16, 4, torch.bfloat16, 5, 4, capi.SCHED_PLANE, 0),
    ("c3", 2, 192, 200, 336, 16, 4, torch.float32, 1, 1, capi.SCHED_STRIPS, 25),
    ("c4", 1, 256, 512, 512, 16, 4, torch.bfloat16, 0, 1, capi.SCHED_STRIPS, 64),
]


@pytest.mark.parametrize("name,Bt,Dm,H,W,N,K,dtype,ob,og,fwd_auto,bwd_jobs", FULL)
def test_full_size_configuration(gpu_device, name, Bt, Dm, H, W, N, K, dtype, ob, og, fwd_auto, bwd_jobs):
    print("full size", name, flush=True)
    dev = gpu_device
    g = torch.Generator(device=dev).manual_seed(1234)
    rn = lambda *s: torch.randn(*s, device=dev, generator=g)
    u, delta = rn(Bt, Dm, H, W).to(dtype), (0.1 * rn(Bt, Dm, H, W)).to(dtype)
    B, Cc = rn(Bt, K, N, H, W).to(dtype), rn(Bt, K, N, H, W).to(dtype)
    dout = rn(Bt, Dm, H, W)
    A = -torch.exp(0.5 * rn(Dm, N))
    D = rn(Dm)
    bias = torch.log(torch.expm1(torch.exp(torch.empty(Dm, device=dev).uniform_(np.log(1e-3), np.log(1e-1), generator=g))))
    args = (u, delta, A, B, Cc, D, bias)

    res = {}
    for sched in (capi.SCHED_AUTO, capi.SCHED_PLANE):
        f = capi.FwdCall(*args, True, True, None, True, sched)
        f.launch()
        b = capi.BwdCall(*args, dout, f.x, f.x_v, True, None, f.x_sd, sched)
        b.launch()
        torch.cuda.synchronize()
        if sched == capi.SCHED_AUTO:
            assert f.plan.auto_schedule == fwd_auto and f.plan.auto_bwd_jobs == bwd_jobs
            if fwd_auto != capi.SCHED_PLANE:               # a whole-plane launch leaves the workspace alone
                assert int(f.ws.view(torch.int32)[1]) == 0, "a forward strip wait ran into its poll limit"
            if bwd_jobs != 0:
                assert int(b.ws.view(torch.int32)[1]) == 0, "a backward strip wait ran into its poll limit"
        res[sched] = (f.out, b.du, b.ddelta, b.dA, b.dB, b.dC, b.dD, b.dbias)
        del f, b
    auto, plane = res[capi.SCHED_AUTO], res[capi.SCHED_PLANE]
    for i in range(3):
        assert torch.equal(auto[i], plane[i]), i
    for i in range(3, 8):
        assert relerr(auto[i].cpu().numpy(), plane[i].cpu().numpy()) <= 1e-5, i

    # oracle on one batch image (and its first `og` channel groups), on the values the kernels saw
    rg = Dm // K
    cs = slice(0, og * rg)
    f32 = lambda t_: t_.float().cpu().numpy()
    o = (f32(u[ob:ob + 1, cs]), f32(delta[ob:ob + 1, cs]), f32(A[cs]), f32(B[ob:ob + 1, :og]), f32(Cc[ob:ob + 1, :og]),
         f32(D[cs]), f32(bias[cs]))
    ref = OC.fwd(*o, True, None, real="f64")
    gref = OC.bwd(*o, f32(dout[ob:ob + 1, cs]), True, None, real="f64")
    half = dtype != torch.float32
    assert relerr(f32(auto[0][ob:ob + 1, cs]), ref) <= 1e-4
    tol = 1e-2 if half else 2e-4
    assert relerr(f32(auto[1][ob:ob + 1, cs]), gref[0]) <= tol          # du
    assert relerr(f32(auto[2][ob:ob + 1, cs]), gref[1]) <= tol          # ddelta
    assert relerr(f32(auto[4][ob:ob + 1, :og]), gref[3]) <= tol         # dB
    assert relerr(f32(auto[5][ob:ob + 1, :og]), gref[4]) <= tol         # dC
