"""Wide planes.  Under the row-segment wavefront kernels (1-4 states, more than eight 64-column segments per row) the
segments are taken in column groups of eight, one launch per group, and what crosses a group boundary goes through
memory.  Under the tile kernels planes wider than 1024 columns are the reference's nChunksX > 1 path
(selective_scan_oflex.cpp:249): many column tiles per strip, the out gather over groups of tiles, hand-over rows at
hundreds of tiles.  Against the float64 oracle on the same inputs, through the C ABI and through the autograd function."""
import numpy as np
import pytest
import torch

import capi
from oracle import snd_oracle as O
from test_gpu_fwd import relerr
from test_gpu_wave import NAMES, check_against_oracle, run

pytestmark = pytest.mark.gpu

WIDE = [
    # Bt, Dm, H, W, N, K, Dd, dtype, kw
    (1, 8, 9, 1500, 2, 2, None, torch.float32, {}),                    # 24 segments: three groups of eight
    (1, 4, 8, 601, 1, 1, None, torch.float32, {}),                     # odd width, one state: ten segments, 8 + 2
    (1, 4, 13, 1100, 1, 1, None, torch.float32, {}),                   # one state beyond 1024 columns: 18 segments, 8 + 8 + 2
    (2, 6, 11, 700, 3, 2, None, torch.bfloat16, {}),                   # three states, 11 segments
    (1, 8, 10, 520, 4, 4, 4, torch.float32, dict(dirs=capi.DIR_CORNERS)),   # nine segments: the second group is one wave
    (1, 4, 1, 1300, 2, 2, None, torch.float32, {}),                    # a single row: a 1D scan through three groups
    (1, 8, 21, 1024, 2, 4, None, torch.float16, dict(decay=0.9)),      # whole segments, whole groups
    (2, 8, 6, 2000, 1, 4, None, torch.bfloat16, dict(dirs=capi.DIR_CORNERS, softplus=False)),
    (1, 4, 7, 900, 2, 2, None, torch.bfloat16, dict(out_float=False)),
    (1, 8, 5, 640, 4, 2, None, torch.float32, dict(use_D=False, use_bias=False)),
]


@pytest.mark.parametrize("Bt,Dm,H,W,N,K,Dd,dtype,kw", WIDE)
def test_wide_planes_match_oracle(gpu_device, Bt, Dm, H, W, N, K, Dd, dtype, kw):
    print("wide", Bt, Dm, H, W, N, K, Dd, dtype, kw, flush=True)
    d, t, f, b = run(gpu_device, Bt, Dm, H, W, N, K, Dd, dtype, capi.SCHED_WAVEFRONT, **kw)
    assert f.plan.wavefront_workspace == 1
    check_against_oracle(d, t, f, b, Dd=Dd, **kw)


@pytest.mark.parametrize("N,dtype,sched", [(16, torch.float32, capi.SCHED_PLANE), (16, torch.float32, capi.SCHED_STRIPS),
                                           (4, torch.float32, capi.SCHED_STRIPS), (16, torch.bfloat16, capi.SCHED_STRIPS),
                                           (1, torch.float32, capi.SCHED_PLANE), (12, torch.float32, capi.SCHED_AUTO)])
def test_wide_plane_tile_kernels(gpu_device, N, dtype, sched):
    print("wide plane, tile kernels", N, dtype, sched, flush=True)
    d, t, f, b = run(gpu_device, 1, 8, 9, 1500, N, 2, None, dtype, sched, seed=31)
    assert f.plan.wavefront_workspace == (1 if N <= 4 else 0)
    check_against_oracle(d, t, f, b)


def test_wide_forward_without_saved_state_and_static_backward(gpu_device):
    """A forward that saves no state hands over between the column groups through its workspace (and, under AUTO with no
    workspace, runs the tile kernels); the backward through the library's static scratch equals the one through a
    caller workspace."""
    Bt, Dm, H, W, N, K = 1, 8, 12, 1200, 2, 4
    d, t, f, b = run(gpu_device, Bt, Dm, H, W, N, K, None, torch.float32, capi.SCHED_WAVEFRONT)
    args = (t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"])
    f2 = capi.FwdCall(*args, True, True, None, False, capi.SCHED_WAVEFRONT)
    f2.launch()
    torch.cuda.synchronize()
    assert f2.x is None
    assert torch.equal(f2.out, f.out)
    stream = torch.cuda.current_stream().cuda_stream
    f2.params.workspace, f2.params.workspace_bytes = None, 0
    assert capi.lib().snd_fwd(capi.C.byref(f2.params), stream) == -6       # WAVEFRONT named: nowhere to hand over
    f2.params.schedule = capi.SCHED_AUTO
    f2.out.zero_()
    assert capi.lib().snd_fwd(capi.C.byref(f2.params), stream) == 0        # AUTO: the tile kernels
    torch.cuda.synchronize()
    assert relerr(f2.out.cpu().numpy(), f.out.cpu().numpy()) <= 1e-5
    want = [x.clone() if x is not None else None for x in (b.du, b.ddelta, b.dA, b.dB, b.dC, b.dD, b.dbias)]
    b.launch_static()
    torch.cuda.synchronize()
    for nm, a, w_ in zip(NAMES, (b.du, b.ddelta, b.dA, b.dB, b.dC, b.dD, b.dbias), want):
        assert relerr(a.float().cpu().numpy(), w_.float().cpu().numpy()) <= 1e-5, nm
    b.params.workspace, b.params.workspace_bytes = None, 0
    assert capi.lib().snd_bwd(capi.C.byref(b.params), stream) == -6


def test_wide_planes_auto_and_autograd(gpu_device):
    """AUTO gives a wide few-state plane to the row-segment kernels, and the autograd function (which allocates the
    backward's workspace itself) returns the oracle's gradients."""
    import selective_nd_scan as snd
    Bt, Dm, H, W, N, K = 1, 8, 16, 1030, 2, 4
    d = O.make_inputs(Bt, Dm, H, W, N=N, K=K, seed=5)
    st, plan = capi.make_plan(capi.Shape(Bt, Dm, H, W, N, K, Dm, capi.SND_F32))
    assert st == 0 and plan.auto_schedule == capi.SCHED_WAVEFRONT and plan.wavefront_workspace == 1
    t = {k: torch.from_numpy(v).to(gpu_device) for k, v in d.items()}
    leaves = [t[k].clone().requires_grad_(True) for k in ("u", "delta", "A", "B", "C", "D", "delta_bias")]
    out = snd.selective_nd_scan(*leaves, delta_softplus=True)
    out.backward(t["dout"])
    torch.cuda.synchronize()
    from oracle_ref import reference
    ref, gref = reference(d["u"], d["delta"], d["A"], d["B"], d["C"], d["D"], d["delta_bias"], d["dout"], True, None, False)
    assert relerr(out.detach().cpu().numpy(), ref) <= 1e-4
    for nm, leaf, w_ in zip(NAMES, leaves, gref):
        assert relerr(leaf.grad.cpu().numpy(), w_) <= 1e-4, nm
