"""fwd + bwd captured in a HIP graph (every schedule): every replay, with eager work and
synchronisations in between, must reproduce the eager result.  The library itself records only
kernels (its sync words are cleared by a fill kernel, not a memset node)."""
import pytest
import torch

import capi
from oracle import snd_oracle as O
from test_gpu_fwd import relerr

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("sched,dims", [(capi.SCHED_PLANE, (2, 16, 40, 24, 16)), (capi.SCHED_STRIPS, (2, 16, 40, 24, 16)),
                                        (capi.SCHED_BANDS, (2, 16, 40, 24, 16)),
                                        # the row-segment kernels: packed planes in four-wave blocks; three segments
                                        (capi.SCHED_WAVEFRONT, (4, 160, 14, 14, 1)), (capi.SCHED_WAVEFRONT, (2, 16, 40, 150, 2)),
                                        # a wide plane: three launches per kernel (column groups) handing over through memory
                                        (capi.SCHED_WAVEFRONT, (1, 8, 12, 1300, 2)),
                                        # split planes: two halves of a plane side by side, tagged words between them (backward)
                                        (capi.SCHED_WAVEFRONT, (1, 128, 9, 512, 1)),
                                        # strips of the 16-lane backward cut into three column segments (forced)
                                        (-3, (2, 16, 40, 100, 16))])
def test_graph_replays_match_eager(gpu_device, sched, dims):
    print("graph", sched, dims, flush=True)
    segments = 0
    if sched < 0:
        segments, sched = -sched, capi.SCHED_STRIPS
    capi.lib().snd_debug_set_strip_slots(-segments)
    try:
        _graph_replays(gpu_device, sched, dims)
    finally:
        capi.lib().snd_debug_set_strip_slots(0)


def _graph_replays(gpu_device, sched, dims):
    d = O.make_inputs(*dims[:4], N=dims[4], K=4, seed=13)
    t = {k: torch.from_numpy(v).to(gpu_device) for k, v in d.items()}
    args = (t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"])

    def run(f, b, stream):
        f.launch(stream)
        b.zero()
        b.launch_kernel_only(stream)

    # eager reference
    f0 = capi.FwdCall(*args, True, True, None, True, sched)
    b0 = capi.BwdCall(*args, t["dout"], f0.x, f0.x_v, True, None, f0.x_sd, sched)
    run(f0, b0, None)
    torch.cuda.synchronize()
    want = [f0.out.clone(), b0.du.clone(), b0.ddelta.clone(), b0.dA.clone(), b0.dB.clone(), b0.dC.clone()]

    f = capi.FwdCall(*args, True, True, None, True, sched)
    b = capi.BwdCall(*args, t["dout"], f.x, f.x_v, True, None, f.x_sd, sched)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(f, b, side.cuda_stream)                      # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        run(f, b, torch.cuda.current_stream().cuda_stream)
    for rep in range(4):
        for o in (f.out, b.du, b.ddelta):
            o.fill_(float("nan"))                        # eager work between replays
        scratch = torch.randn(1 << 16, device=gpu_device).sum().item()
        g.replay()
        torch.cuda.synchronize()
        got = [f.out, b.du, b.ddelta, b.dA, b.dB, b.dC]
        for i, (a, w) in enumerate(zip(got, want)):
            tol = 0.0 if i < 3 else 1e-5                 # atomic sums may differ in order
            assert relerr(a.cpu().numpy(), w.cpu().numpy()) <= tol, (rep, i)
        if sched not in (capi.SCHED_PLANE, capi.SCHED_WAVEFRONT):
            assert int(f.ws.view(torch.int32)[1]) == 0 and int(b.ws.view(torch.int32)[1]) == 0
        elif sched == capi.SCHED_WAVEFRONT and f.plan.wavefront_workspace:
            assert int(b.ws.view(torch.int32)[1]) == 0   # no hand-over wait of a wide or split plane gave up
