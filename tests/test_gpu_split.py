"""Split planes in the row-segment backward: few planes (at most 256) of eight row segments with one or two
states are cut in two halves that run side by side, two channels per block, and hand the adjoint of the middle column
over through tagged words in the workspace.  Against the float64 oracle, against the same kernel family without the
split (no workspace given), and with the hand-over's bounded wait cut short from the host."""
import numpy as np
import pytest
import torch

import capi
from test_gpu_fwd import relerr
from test_gpu_wave import NAMES, check_against_oracle, run

pytestmark = pytest.mark.gpu

SPLIT = [
    # Bt, Dm, H, W, N, K, Dd, dtype, kw        (planes * segments >= 1024, planes <= 256)
    (1, 128, 9, 512, 1, 4, None, torch.float32, {}),                               # eight whole segments, two whole bands + 1 row
    (2, 96, 10, 512, 2, 4, None, torch.bfloat16, {}),                              # two states, whole bands and segments
    (1, 132, 7, 500, 1, 4, None, torch.float32, dict(dirs=capi.DIR_CORNERS)),     # 33 channels per group: the last block repeats one
    (1, 256, 6, 450, 1, 4, 128, torch.float16, dict(decay=0.9)),                   # 256 planes, ragged last segment, shared delta
    (1, 192, 5, 458, 2, 2, None, torch.float32, dict(softplus=False)),             # the last segment 10 columns wide
    (1, 128, 1, 512, 2, 4, None, torch.float32, {}),                               # a single row
    (1, 128, 12, 512, 1, 4, None, torch.bfloat16, dict(out_float=False)),          # whole bands and segments, one state
]


@pytest.mark.parametrize("Bt,Dm,H,W,N,K,Dd,dtype,kw", SPLIT)
def test_split_planes_match_oracle_and_whole_planes(gpu_device, Bt, Dm, H, W, N, K, Dd, dtype, kw):
    print("split", Bt, Dm, H, W, N, K, Dd, dtype, kw, flush=True)
    d, t, f, b = run(gpu_device, Bt, Dm, H, W, N, K, Dd, dtype, capi.SCHED_WAVEFRONT, **kw)
    assert f.plan.wavefront_workspace == 1
    assert int(b.ws.view(torch.int32)[1]) == 0          # no hand-over wait gave up
    check_against_oracle(d, t, f, b, Dd=Dd, **kw)
    # the same backward without a workspace: whole planes, one channel per block
    got = [x.clone() if x is not None else None for x in (b.du, b.ddelta, b.dA, b.dB, b.dC, b.dD, b.dbias, b.ddec)]
    b.params.workspace, b.params.workspace_bytes = None, 0
    b.launch()
    torch.cuda.synchronize()
    half = dtype != torch.float32
    for nm, a, w_ in zip(NAMES, got, (b.du, b.ddelta, b.dA, b.dB, b.dC, b.dD, b.dbias, b.ddec)):
        assert (a is None) == (w_ is None), nm
        if a is None:
            continue
        tol = 1e-2 if (half and nm in ("du", "ddelta")) else (5e-4 if nm == "dA_decay" else 1e-4)
        assert relerr(a.float().cpu().numpy(), w_.float().cpu().numpy()) <= tol, nm


def test_split_planes_wait_is_bounded(gpu_device):
    """With the wait for the other half cut to one poll the launch still ends; a half that gave up has set the error
    word and returns NaN, never plausible numbers; otherwise the result is the usual one."""
    d, t, f, b = run(gpu_device, 1, 128, 12, 512, 1, 4, None, torch.float32, capi.SCHED_WAVEFRONT)
    want = b.du.clone()
    capi.lib().snd_debug_set_spin_limit(1)
    try:
        b.launch()
        torch.cuda.synchronize()
    finally:
        capi.lib().snd_debug_set_spin_limit(0)
    gave_up = int(b.ws.view(torch.int32)[1]) != 0
    if gave_up:
        assert torch.isnan(b.du).any()
        assert capi.lib().snd_workspace_error(b.ws.data_ptr(), torch.cuda.current_stream().cuda_stream) == -9
    else:
        assert torch.equal(b.du, want)
    b.launch()                                           # and the next launch on the same workspace is clean
    torch.cuda.synchronize()
    assert int(b.ws.view(torch.int32)[1]) == 0
    assert torch.equal(b.du, want)
