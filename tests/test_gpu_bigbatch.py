"""Tensors larger than 4 GiB: offsets across batch images are 64-bit in both kernel families (the reference
indexes with 32-bit strides inside a batch image and 64-bit products across it, selective_scan_oflex.cpp:37-110).
u, delta, out, du and ddelta of these cases span 2^32 bytes or more; one launch over the whole batch must
give what two launches over its halves give (no CPU oracle: the halves are the reference here, and each
half stays below 2^32 bytes per tensor)."""
import pytest
import torch

import capi
from test_gpu_fwd import relerr

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("N", [5, 1])      # 5: the tile kernels (eight lanes per channel); 1: the row-segment kernels
def test_batch_offsets_beyond_4gib(gpu_device, N):
    print("big batch", N, flush=True)
    free, _ = torch.cuda.mem_get_info()
    if free < 80 * 2 ** 30:
        pytest.skip("needs about 60 GiB of device memory")
    Bt, Dm, H, W, K = 4096, 64, 64, 64, 1
    g = torch.Generator(device=gpu_device)
    g.manual_seed(7)
    rn = lambda *s: torch.randn(*s, device=gpu_device, generator=g)
    u, delta, dout = rn(Bt, Dm, H, W), 0.1 * rn(Bt, Dm, H, W), rn(Bt, Dm, H, W)
    assert u.numel() * u.element_size() >= 2 ** 32
    A = -torch.exp(0.5 * rn(Dm, N))
    B, C = rn(Bt, K, N, H, W), rn(Bt, K, N, H, W)
    D, bias = rn(Dm), -4.0 + rn(Dm)

    def run(lo, hi):
        args = (u[lo:hi], delta[lo:hi], A, B[lo:hi], C[lo:hi], D, bias)
        f = capi.FwdCall(*args, True, True, None, True, capi.SCHED_AUTO)
        f.launch()
        b = capi.BwdCall(*args, dout[lo:hi], f.x, f.x_v, True, None, f.x_sd, capi.SCHED_AUTO)
        b.launch()
        torch.cuda.synchronize()
        return f.out, b.du, b.ddelta, b.dB, b.dC, b.dA, b.dD, b.dbias

    full = run(0, Bt)
    # the last images of the batch sit beyond 2^32 bytes in the full run and near the start of the second half's
    acc = None
    for lo, hi in ((0, Bt // 2), (Bt // 2, Bt)):
        part = run(lo, hi)
        for i in range(3):                                   # out, du, ddelta: written once, bit-identical
            assert torch.equal(full[i][lo:hi], part[i]), ("out", "du", "ddelta")[i]
        for i in (3, 4):                                     # dB, dC: per image, summed over channels with atomics
            assert relerr(full[i][lo:hi].cpu().numpy(), part[i].cpu().numpy()) <= 1e-5, ("dB", "dC")[i - 3]
        small = [t.double() for t in part[5:]]
        acc = small if acc is None else [a + s for a, s in zip(acc, small)]
        del part
    for nm, a, w in zip(("dA", "dD", "ddelta_bias"), full[5:], acc):
        assert relerr(a.cpu().numpy(), w.cpu().numpy()) <= 1e-4, nm
