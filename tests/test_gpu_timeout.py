"""The time-out path of the pipelined schedules, forced from the host: with a poll limit of one, any
hand-over wait that is not already satisfied gives up.  Every kernel still runs to completion; a block
that gave up sets the workspace's error word and poisons what it computes with NaN, so a caller can
never mistake the result for a good one, and snd_workspace_error reports it."""
import numpy as np
import pytest
import torch

import capi
from oracle import snd_oracle as O
from oracle import snd_oracle_c as OC
from test_gpu_fwd import relerr

pytestmark = pytest.mark.gpu


def test_forced_timeout_is_loud(gpu_device):
    print("forced hand-over time-out", flush=True)
    lib = capi.lib()
    d = O.make_inputs(1, 32, 160, 160, N=16, K=2, seed=13)       # 2 plane chunks x 20 strips x 20 tiles
    t = {k: torch.from_numpy(v).to(gpu_device) for k, v in d.items()}
    args = (t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"])
    ref = OC.fwd(d["u"], d["delta"], d["A"], d["B"], d["C"], d["D"], d["delta_bias"], True, None, real="f64")
    stream = torch.cuda.current_stream().cuda_stream
    try:
        lib.snd_debug_set_spin_limit(1)
        f = capi.FwdCall(*args, True, True, None, True, capi.SCHED_STRIPS)
        f.launch()
        torch.cuda.synchronize()
        st = lib.snd_workspace_error(f.ws.data_ptr(), stream)
        word = int(f.ws.view(torch.int32)[1])
        out = f.out.cpu().numpy()
        if word:
            assert st == -9 and np.isnan(out).any(), "a timed-out launch must report it and poison its outputs"
        else:                                                    # every wait happened to be satisfied at once
            assert st == 0 and relerr(out, ref) <= 1e-4
    finally:
        lib.snd_debug_set_spin_limit(0)
    # with the default limit the same launch is clean
    f = capi.FwdCall(*args, True, True, None, True, capi.SCHED_STRIPS)
    f.launch()
    b = capi.BwdCall(*args, t["dout"], f.x, f.x_v, True, None, f.x_sd, capi.SCHED_STRIPS)
    b.launch()
    torch.cuda.synchronize()
    assert lib.snd_workspace_error(f.ws.data_ptr(), stream) == 0
    assert lib.snd_workspace_error(b.ws.data_ptr(), stream) == 0
    assert relerr(f.out.cpu().numpy(), ref) <= 1e-4 and not torch.isnan(b.du).any()


def test_extension_debug_check_raises_on_timeout(gpu_device):
    import selective_nd_scan as snd
    lib = capi.lib()
    d = O.make_inputs(1, 32, 160, 160, N=16, K=2, seed=14, with_dout=False)
    t = {k: torch.from_numpy(v).to(gpu_device) for k, v in d.items()}
    args = (t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"], True, True, None)
    try:
        snd.set_debug(True)
        snd.fwd(*args, schedule=capi.SCHED_STRIPS)               # clean: must not raise
        lib.snd_debug_set_spin_limit(1)
        raised = False
        for _ in range(3):
            try:
                out = snd.fwd(*args, schedule=capi.SCHED_STRIPS)[0]
            except RuntimeError as e:
                assert "timed out" in str(e)
                raised = True
                break
            assert not torch.isnan(out).any()                    # no time-out happened: then the result is clean
        print("debug check raised:", raised, flush=True)
    finally:
        lib.snd_debug_set_spin_limit(0)
        snd.set_debug(False)
