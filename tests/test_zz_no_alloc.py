"""snd_bwd_static - the backward for callers that cannot allocate: same kernels as snd_bwd, scratch in
the library's static device array instead of a caller workspace.  Two calls in a row through the C ABI,
the second on a smaller problem (it must not be disturbed by what the first left in the shared array),
each compared with snd_bwd on the same inputs and with the float64 oracle."""
import pytest
import torch

import capi
from oracle import snd_oracle as O
from oracle import snd_oracle_c as OC
from test_gpu_fwd import relerr

pytestmark = pytest.mark.gpu
NAMES = ["du", "ddelta", "dA", "dB", "dC", "dD", "ddelta_bias"]


def _case(dev, Bt, Dm, H, W, N, K, sched, seed):
    d = O.make_inputs(Bt, Dm, H, W, N=N, K=K, seed=seed)
    t = {k: torch.from_numpy(v).to(dev) for k, v in d.items()}
    args = (t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"])
    f = capi.FwdCall(*args, True, True, None, True, sched)
    f.launch()
    b = capi.BwdCall(*args, t["dout"], f.x, f.x_v, True, None, f.x_sd, sched)
    return d, t, f, b


def _grads(b):
    return [x.clone() for x in (b.du, b.ddelta, b.dA, b.dB, b.dC, b.dD, b.dbias)]


def test_bwd_static_matches_bwd_twice_second_smaller(gpu_device):
    print("no-alloc backward: two calls, second smaller", flush=True)
    lib = capi.lib()
    assert lib.snd_init(0) == 0
    # first call: pipelined strips (uses the sync words and the hand-over rows of the scratch);
    # second call: a smaller problem with whole-plane blocks (uses the adjoint rows only)
    for (Bt, Dm, H, W, N, K, sched, seed) in [(2, 32, 40, 24, 16, 4, capi.SCHED_STRIPS, 7),
                                              (1, 16, 17, 9, 16, 2, capi.SCHED_PLANE, 8)]:
        d, t, f, b = _case(gpu_device, Bt, Dm, H, W, N, K, sched, seed)
        b.launch()                                   # snd_bwd with a caller workspace
        torch.cuda.synchronize()
        want = _grads(b)
        count = lambda: torch.cuda.memory_stats()["allocation.all.allocated"]   # allocations made so far (cumulative)
        before = count()
        b.launch_static()                            # snd_bwd_static: no workspace passed
        torch.cuda.synchronize()
        assert count() == before, "the call allocated device memory through torch"
        got = _grads(b)
        # same kernels, same arithmetic: everything that is not an atomic sum is bit-identical
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
        for nm, a, w in zip(NAMES[2:], got[2:], want[2:]):
            assert relerr(a.cpu().numpy(), w.cpu().numpy()) <= 1e-5, nm
        gref = OC.bwd(d["u"], d["delta"], d["A"], d["B"], d["C"], d["D"], d["delta_bias"], d["dout"], True, None, real="f64")
        for nm, a, r in zip(NAMES, got, gref):
            assert relerr(a.cpu().numpy(), r) <= 1e-4, (nm, relerr(a.cpu().numpy(), r))


def test_bwd_static_refuses_what_does_not_fit(gpu_device):
    d, t, f, b = _case(gpu_device, 1, 8, 9, 10, 16, 2, capi.SCHED_AUTO, 3)
    q = capi.BwdParams.from_buffer_copy(b.params)
    q.f.shape = capi.Shape(64, 768, 56, 56, 16, 4, 768, capi.SND_F32)
    assert capi.lib().snd_bwd_static(capi.C.byref(q), torch.cuda.current_stream().cuda_stream) == -8
    # the same size with one state runs the row-segment kernels, which use no scratch: never refused for size
    # (null inputs: the call must get past the size check and stop at the pointer checks instead)
    q.f.shape = capi.Shape(64, 768, 56, 56, 1, 4, 768, capi.SND_F32)
    q.f.u = None
    assert capi.lib().snd_bwd_static(capi.C.byref(q), torch.cuda.current_stream().cuda_stream) == -1


def test_bwd_static_few_states_and_timeout_query(gpu_device):
    """AUTO with one state (row-segment kernels) through the static entry point, and the error word of the static
    scratch read back through snd_workspace_error(NULL, stream): clean after a clean pipelined call, set after one
    whose hand-over waits were forced to give up (poll limit 1; every kernel still drains, the outputs are NaN)."""
    lib = capi.lib()
    stream = torch.cuda.current_stream().cuda_stream
    d, t, f, b = _case(gpu_device, 2, 16, 30, 70, 1, 4, capi.SCHED_AUTO, 5)
    b.launch()
    torch.cuda.synchronize()
    want = _grads(b)
    b.launch_static()
    torch.cuda.synchronize()
    got = _grads(b)
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
    for nm, a, w in zip(NAMES[2:], got[2:], want[2:]):
        assert relerr(a.cpu().numpy(), w.cpu().numpy()) <= 1e-5, nm
    d, t, f, b = _case(gpu_device, 1, 32, 160, 160, 16, 2, capi.SCHED_STRIPS, 13)
    b.launch_static()
    torch.cuda.synchronize()
    assert lib.snd_workspace_error(None, stream) == 0 and not torch.isnan(b.du).any()
    try:
        lib.snd_debug_set_spin_limit(1)
        b.launch_static()
        torch.cuda.synchronize()
        st = lib.snd_workspace_error(None, stream)
        assert st in (0, -9)
        if st == -9:
            assert torch.isnan(b.du).any(), "a timed-out launch must poison its outputs"
        else:                                         # every wait happened to be satisfied at once
            assert not torch.isnan(b.du).any()
    finally:
        lib.snd_debug_set_spin_limit(0)
    b.launch_static()
    torch.cuda.synchronize()
    assert lib.snd_workspace_error(None, stream) == 0 and not torch.isnan(b.du).any()
