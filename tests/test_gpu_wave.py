"""The row-segment wavefront kernels (1-4 states per channel, planes of at most eight row segments) against the
float64 oracle and against the tile kernels on the same inputs, through the C ABI."""
import numpy as np
import pytest
import torch

import capi
from oracle import snd_oracle as O
from oracle import snd_oracle_c as OC
from oracle_ref import reference
from test_gpu_fwd import relerr

pytestmark = pytest.mark.gpu
NAMES = ["du", "ddelta", "dA", "dB", "dC", "dD", "ddelta_bias", "dA_decay"]

SHAPES = [
    # Bt, Dm, H, W, N, K, Dd, dtype
    (1, 8, 9, 10, 1, 2, None, torch.float32),        # one segment, partly filled
    (2, 8, 16, 64, 1, 4, None, torch.float32),       # exactly one full segment, two full bands
    (1, 4, 17, 65, 1, 1, None, torch.float32),       # second segment holds one column; ragged last band
    (1, 4, 1, 200, 2, 2, None, torch.float32),       # single row: 1D scan across four segments
    (1, 4, 33, 1, 2, 1, None, torch.float32),        # single column
    (1, 8, 30, 130, 2, 4, 4, torch.float32),         # three segments, shared delta groups
    (2, 6, 21, 100, 3, 2, None, torch.float32),      # three states
    (1, 8, 13, 150, 4, 2, None, torch.float32),      # four states: bands of four rows
    (1, 8, 40, 512, 1, 4, None, torch.float32),      # the widest plane: eight segments
    (1, 8, 64, 512, 1, 4, None, torch.bfloat16),
    (3, 12, 14, 14, 4, 4, None, torch.bfloat16),
    (1, 4, 25, 90, 2, 2, None, torch.float16),
    (2, 48, 56, 56, 1, 4, None, torch.float32),      # stage-1 plane, d_state = 1
    # one state and an even width above 64: two neighbouring columns per lane
    (1, 4, 19, 66, 1, 2, None, torch.float32),       # 33 lanes of one wave
    (1, 8, 17, 130, 1, 4, None, torch.float32),      # second segment holds one lane
    (2, 8, 33, 256, 1, 4, 4, torch.bfloat16),        # two full segments, shared delta groups
    (1, 4, 12, 1024, 1, 1, None, torch.float16),     # the widest plane: eight segments of 128 columns
    (1, 8, 70, 200, 1, 4, None, torch.bfloat16),
    # more blocks of 4 to 8 waves than fit at three waves per SIMD: the forward's instantiation with room for four
    (2, 192, 20, 300, 1, 4, None, torch.float32),
    (4, 256, 16, 256, 2, 4, None, torch.bfloat16),
    # group counts that are no power of two (the pair -> (batch, group) split divides), with 18 and 30 pairs dealt to
    # the XCDs and 3 pairs not; one-segment planes whose channels do not fill the forward's blocks of four waves
    (6, 15, 9, 20, 1, 3, None, torch.float32),
    (6, 30, 11, 70, 2, 5, 15, torch.bfloat16),
    (1, 18, 6, 12, 1, 3, 9, torch.float32),
]


def run(dev, Bt, Dm, H, W, N, K, Dd, dtype, sched, dirs=capi.DIR_TOPLEFT, softplus=True, decay=None, seed=3,
        use_D=True, use_bias=True, out_float=True):
    d = O.make_inputs(Bt, Dm, H, W, N=N, K=K, seed=seed, Dd=Dd)
    t = {k: torch.from_numpy(v).to(dev) for k, v in d.items()}
    for k in ("u", "delta", "B", "C"):
        t[k] = t[k].to(dtype)
    if not softplus:                                  # a raw delta must be positive: pass the discretised step itself
        t["delta"] = torch.nn.functional.softplus(t["delta"].float() + t["delta_bias"].view(1, -1, 1, 1).repeat_interleave(Dm // t["delta"].shape[1], 1)[:, :t["delta"].shape[1]]).to(dtype)
        d["delta"] = t["delta"].float().cpu().numpy()
        use_bias = False
    D = t["D"] if use_D else None
    bias = t["delta_bias"] if use_bias else None
    dec = torch.tensor([decay], device=dev) if decay is not None else None
    args = (t["u"], t["delta"], t["A"], t["B"], t["C"], D, bias)
    f = capi.FwdCall(*args, softplus, out_float, dec, True, sched, dirs)
    f.launch()
    b = capi.BwdCall(*args, t["dout"], f.x, f.x_v, softplus, dec, f.x_sd, sched, dirs)
    b.launch()
    torch.cuda.synchronize()
    return d, t, f, b


def check_against_oracle(d, t, f, b, Dd=None, softplus=True, decay=None, dirs=capi.DIR_TOPLEFT, use_D=True, use_bias=True,
                         out_float=True, **_):
    """The run's out and all eight gradients against the float64 oracle on the values the kernels saw, with the
    run's options (corner directions by flipped copies).  fp32: 1e-4 (dA_decay 5e-4: a single number whose terms
    cancel to a few percent of their size); 16-bit inputs: 1e-2 on the tensors stored in 16 bits."""
    r = {k: t[k].float().cpu().numpy() for k in ("u", "delta", "B", "C")}
    use_bias = use_bias and softplus
    ref, gref = reference(r["u"], r["delta"], d["A"], r["B"], r["C"], d["D"] if use_D else None,
                          d["delta_bias"] if use_bias else None, d["dout"], softplus, decay, dirs == capi.DIR_CORNERS)
    half = t["u"].dtype != torch.float32
    Bt, Dm, H, W = t["u"].shape[0], d["A"].shape[0], t["u"].shape[2], t["u"].shape[3]
    assert relerr(f.out.float().cpu().numpy(), ref) <= (1e-2 if not out_float else 1e-4)
    got = [b.du, b.ddelta, b.dA, b.dB, b.dC, b.dD, b.dbias, b.ddec]
    if Dd is not None:                                # the C ABI returns ddelta / ddelta_bias per channel
        got[1] = got[1].float().view(Bt, Dd, Dm // Dd, H, W).sum(2)
        if got[6] is not None:
            got[6] = got[6].view(Dd, Dm // Dd).sum(1)
    for nm, a, w_ in zip(NAMES, got, gref):
        assert (a is None) == (w_ is None), nm
        if a is None:
            continue
        tol = 1e-2 if (half and nm in ("du", "ddelta", "dB", "dC")) else (5e-4 if nm == "dA_decay" else 1e-4)
        e = relerr(a.float().cpu().numpy(), w_)
        assert e <= tol, (nm, e)


@pytest.mark.parametrize("Bt,Dm,H,W,N,K,Dd,dtype", SHAPES)
def test_wavefront_matches_oracle_and_tiles(gpu_device, Bt, Dm, H, W, N, K, Dd, dtype):
    print("wavefront", Bt, Dm, H, W, N, K, Dd, dtype, flush=True)
    d, t, f, b = run(gpu_device, Bt, Dm, H, W, N, K, Dd, dtype, capi.SCHED_WAVEFRONT)
    r = {k: t[k].float().cpu().numpy() for k in ("u", "delta", "B", "C")}
    o = (r["u"], r["delta"], d["A"], r["B"], r["C"], d["D"], d["delta_bias"])
    ref = OC.fwd(*o, True, None, real="f64")
    gref = OC.bwd(*o, d["dout"], True, None, real="f64")
    assert relerr(f.out.cpu().numpy(), ref) <= 1e-4
    half = dtype != torch.float32
    Dmm = Dm
    got = [b.du, b.ddelta, b.dA, b.dB, b.dC, b.dD, b.dbias]
    if Dd is not None:                                # the C ABI returns ddelta / ddelta_bias per channel
        got[1] = got[1].float().view(Bt, Dd, Dmm // Dd, H, W).sum(2)
        got[6] = got[6].view(Dd, Dmm // Dd).sum(1)
    for nm, a, w_ in zip(NAMES, got, gref):
        tol = 1e-2 if (half and nm in ("du", "ddelta", "dB", "dC")) else 1e-4
        e = relerr(a.float().cpu().numpy(), w_)
        assert e <= tol, (nm, e)
    # the tile kernels on the same inputs (their own saved state)
    _, _, f2, b2 = run(gpu_device, Bt, Dm, H, W, N, K, Dd, dtype, capi.SCHED_PLANE)
    assert relerr(f.out.cpu().numpy(), f2.out.cpu().numpy()) <= 1e-5
    got2 = [b2.du, b2.ddelta, b2.dA, b2.dB, b2.dC, b2.dD, b2.dbias]
    if Dd is not None:
        got2[1] = got2[1].float().view(Bt, Dd, Dmm // Dd, H, W).sum(2)
        got2[6] = got2[6].view(Dd, Dmm // Dd).sum(1)
    for nm, a, w_, r_ in zip(NAMES, got, got2, gref):
        # difference of the two kernel families on the scale of the true gradient (a single row makes dA
        # identically zero: both families then return rounding noise of different sizes)
        tol = 1e-2 if (half and nm in ("du", "ddelta")) else 1e-4
        scale = max(float(np.abs(r_).max()), 1e-2 if float(np.abs(r_).max()) < 1e-12 else 0.0)
        e = float(np.abs(a.float().cpu().numpy().astype(np.float64) - w_.float().cpu().numpy()).max()) / scale
        assert e <= tol, (nm, e)


@pytest.mark.parametrize("kw", [dict(softplus=False), dict(use_D=False, use_bias=False), dict(decay=0.9),
                                dict(dirs=capi.DIR_CORNERS), dict(out_float=False)])
def test_wavefront_options(gpu_device, kw):
    print("wavefront options", kw, flush=True)
    Bt, Dm, H, W, N, K = 2, 8, 19, 150, 2, 4
    dtype = torch.bfloat16 if kw.get("out_float") is False else torch.float32
    d, t, f, b = run(gpu_device, Bt, Dm, H, W, N, K, None, dtype, capi.SCHED_WAVEFRONT, **kw)
    _, _, f2, b2 = run(gpu_device, Bt, Dm, H, W, N, K, None, dtype, capi.SCHED_PLANE, **kw)
    half = dtype != torch.float32
    assert f.out.dtype == (torch.float32 if kw.get("out_float", True) else dtype)
    assert relerr(f.out.float().cpu().numpy(), f2.out.float().cpu().numpy()) <= (1e-2 if half else 1e-5)
    pairs = zip(NAMES, [b.du, b.ddelta, b.dA, b.dB, b.dC, b.dD, b.dbias, b.ddec], [b2.du, b2.ddelta, b2.dA, b2.dB, b2.dC, b2.dD, b2.dbias, b2.ddec])
    for nm, a, w_ in pairs:
        assert (a is None) == (w_ is None), nm
        if a is None:
            continue
        tol = 1e-2 if (half and nm in ("du", "ddelta")) else (5e-4 if nm == "dA_decay" else 1e-4)
        assert relerr(a.float().cpu().numpy(), w_.float().cpu().numpy()) <= tol, (nm, relerr(a.float().cpu().numpy(), w_.float().cpu().numpy()))
    check_against_oracle(d, t, f, b, **kw)          # and the float64 oracle under the same options


def test_wavefront_shared_u_and_second_backward(gpu_device):
    """u with dim / n_groups channels shared by the four corner groups; the saved state is read-only."""
    Bt, Cc_, H, W, N, K = 2, 6, 20, 70, 1, 4
    d = O.make_inputs(Bt, K * Cc_, H, W, N=N, K=K, seed=8)
    t = {k: torch.from_numpy(v).to(gpu_device) for k, v in d.items()}
    u1 = t["u"][:, :Cc_].contiguous()
    args = (u1, t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"])
    res = {}
    for sched in (capi.SCHED_WAVEFRONT, capi.SCHED_PLANE):
        f = capi.FwdCall(*args, True, True, None, True, sched, capi.DIR_CORNERS)
        f.launch()
        g1 = capi.bwd(*args, t["dout"], f.x, f.x_v, True, None, f.x_sd, schedule=sched, directions=capi.DIR_CORNERS)
        g2 = capi.bwd(*args, t["dout"], f.x, f.x_v, True, None, f.x_sd, schedule=sched, directions=capi.DIR_CORNERS)
        torch.cuda.synchronize()
        for a, b_ in zip(g1, g2):
            if a is not None:
                assert relerr(b_.cpu().numpy(), a.cpu().numpy()) <= 1e-6
        res[sched] = (f.out, g1)
    assert res[capi.SCHED_WAVEFRONT][1][0].shape == u1.shape
    assert relerr(res[capi.SCHED_WAVEFRONT][0].cpu().numpy(), res[capi.SCHED_PLANE][0].cpu().numpy()) <= 1e-5
    for a, b_ in zip(res[capi.SCHED_WAVEFRONT][1], res[capi.SCHED_PLANE][1]):
        if a is not None:
            assert relerr(a.cpu().numpy(), b_.cpu().numpy()) <= 1e-4


def test_wavefront_refuses_what_it_does_not_cover(gpu_device):
    d = O.make_inputs(1, 4, 8, 60, N=5, K=1, seed=1)        # five states
    t = {k: torch.from_numpy(v).to(gpu_device) for k, v in d.items()}
    f = capi.FwdCall(t["u"], t["delta"], t["A"], t["B"], t["C"], None, None, False, True, None, True, capi.SCHED_WAVEFRONT)
    assert f.plan.auto_schedule != capi.SCHED_WAVEFRONT
    assert capi.lib().snd_fwd(capi.C.byref(f.params), torch.cuda.current_stream().cuda_stream) == -2


@pytest.mark.parametrize("dtype,dirs", [(torch.float32, capi.DIR_TOPLEFT), (torch.bfloat16, capi.DIR_CORNERS), (torch.float32, capi.DIR_CORNERS)])
def test_wavefront_two_columns_per_lane_unaligned_and_flipped(gpu_device, dtype, dirs):
    """One state, even width: rows that do not start at a multiple of two elements (odd row pitch: every lane's
    pair is loaded element by element) and column-reversed groups, against the tile kernels and the oracle."""
    Bt, Dm, H, W, N, K = 1, 8, 21, 150, 1, 4
    d = O.make_inputs(Bt, Dm, H, W, N=N, K=K, seed=17)
    t = {k: torch.from_numpy(v).to(gpu_device) for k, v in d.items()}

    def padded(x):                                    # same values, row pitch W + 1
        buf = torch.zeros(*x.shape[:-1], W + 1, device=x.device, dtype=dtype)
        buf[..., :W] = x.to(dtype)
        return buf[..., :W]
    res = {}
    for name, mk in (("pitch", padded), ("dense", lambda x: x.to(dtype).contiguous())):
        u, delta, B, C = (mk(t[k]) for k in ("u", "delta", "B", "C"))
        dout = mk(t["dout"]).float() if name == "dense" else padded(t["dout"]).float()
        args = (u, delta, t["A"], B, C, t["D"], t["delta_bias"])
        for sched in (capi.SCHED_WAVEFRONT, capi.SCHED_PLANE):
            f = capi.FwdCall(*args, True, True, None, True, sched, dirs)
            f.launch()
            b = capi.BwdCall(*args, dout, f.x, f.x_v, True, None, f.x_sd, sched, dirs)
            b.launch()
            torch.cuda.synchronize()
            res[(name, sched)] = [f.out, b.du, b.ddelta, b.dA, b.dB, b.dC, b.dD, b.dbias]
    half = dtype != torch.float32
    ref = res[("dense", capi.SCHED_PLANE)]
    for key in (("pitch", capi.SCHED_WAVEFRONT), ("dense", capi.SCHED_WAVEFRONT), ("pitch", capi.SCHED_PLANE)):
        for nm, a, w_ in zip(["out"] + NAMES, res[key], ref):
            tol = 1e-2 if (half and nm in ("du", "ddelta")) else 1e-4
            e = relerr(a.float().cpu().numpy(), w_.float().cpu().numpy())
            assert e <= tol, (key, nm, e)
    if dirs == capi.DIR_TOPLEFT:
        r = {k: t[k].to(dtype).float().cpu().numpy() for k in ("u", "delta", "B", "C")}
        refo = OC.fwd(r["u"], r["delta"], d["A"], r["B"], r["C"], d["D"], d["delta_bias"], True, None, real="f64")
        assert relerr(res[("pitch", capi.SCHED_WAVEFRONT)][0].cpu().numpy(), refo) <= 1e-4


SHARED = [
    # Bt, Dm, H, W, N, K, dtype, kw: one segment per plane and 512 planes or more - the backward's blocks hold four channels
    (8, 264, 20, 24, 1, 4, torch.float32, {}),                 # 66 channels per group: the last block of a group repeats two
    (16, 128, 16, 64, 1, 2, torch.bfloat16, {}),               # whole bands, whole segment
    (8, 256, 12, 40, 2, 4, torch.float32, {}),
    (8, 264, 8, 64, 2, 4, torch.bfloat16, {}),
    (4, 516, 10, 33, 3, 4, torch.float32, {}),                 # three states, 129 channels per group
    (4, 512, 9, 20, 4, 4, torch.float16, {}),
    (8, 264, 21, 30, 1, 4, torch.float32, dict(dirs=capi.DIR_CORNERS, decay=0.9)),
    (8, 256, 16, 64, 2, 4, torch.float32, dict(dirs=capi.DIR_CORNERS, softplus=False)),
    # two segments per plane and a full load of waves (2048): blocks of four channels (two with three or four states)
    (4, 264, 12, 100, 1, 4, torch.float32, {}),
    (4, 256, 16, 128, 2, 4, torch.bfloat16, {}),
    (2, 516, 9, 70, 3, 4, torch.float32, {}),
    (4, 264, 13, 90, 1, 4, torch.float32, dict(dirs=capi.DIR_CORNERS, decay=0.9)),
    # three and four segments per plane, one or two states: blocks of two channels
    (4, 264, 9, 200, 1, 4, torch.float32, {}),
    (8, 128, 10, 130, 2, 4, torch.bfloat16, {}),
    (4, 264, 11, 250, 2, 4, torch.float32, dict(dirs=capi.DIR_CORNERS)),
    # five to eight segments per plane and more planes than CUs: two channels in a block of 10 to 16 waves
    (2, 260, 10, 330, 1, 4, torch.float32, {}),                # 65 channels per group: the last block of a group repeats one
    (2, 264, 8, 512, 2, 4, torch.bfloat16, {}),                # whole bands, whole segments
    (1, 516, 9, 450, 1, 4, torch.float32, dict(dirs=capi.DIR_CORNERS, decay=0.9)),
]


@pytest.mark.parametrize("Bt,Dm,H,W,N,K,dtype,kw", SHARED)
def test_wavefront_shared_atomics(gpu_device, Bt, Dm, H, W, N, K, dtype, kw):
    """Backward blocks of four or two channels whose dB / dC contributions meet in LDS: against the tile kernels, and
    against the oracle where it takes the options."""
    print("wavefront shared atomics", Bt, Dm, H, W, N, K, dtype, kw, flush=True)
    d, t, f, b = run(gpu_device, Bt, Dm, H, W, N, K, None, dtype, capi.SCHED_WAVEFRONT, **kw)
    _, _, f2, b2 = run(gpu_device, Bt, Dm, H, W, N, K, None, dtype, capi.SCHED_PLANE, **kw)
    half = dtype != torch.float32
    assert relerr(f.out.cpu().numpy(), f2.out.cpu().numpy()) <= 1e-5
    for nm, a, w_ in zip(NAMES, [b.du, b.ddelta, b.dA, b.dB, b.dC, b.dD, b.dbias, b.ddec], [b2.du, b2.ddelta, b2.dA, b2.dB, b2.dC, b2.dD, b2.dbias, b2.ddec]):
        assert (a is None) == (w_ is None), nm
        if a is None:
            continue
        tol = 1e-2 if (half and nm in ("du", "ddelta")) else (5e-4 if nm == "dA_decay" else 1e-4)
        e = relerr(a.float().cpu().numpy(), w_.float().cpu().numpy())
        assert e <= tol, (nm, e)
    if not kw:
        r = {k: t[k].float().cpu().numpy() for k in ("u", "delta", "B", "C")}
        o = (r["u"], r["delta"], d["A"], r["B"], r["C"], d["D"], d["delta_bias"])
        gref = OC.bwd(*o, d["dout"], True, None, real="f64")
        for nm, a, w_ in zip(NAMES, [b.du, b.ddelta, b.dA, b.dB, b.dC, b.dD, b.dbias], gref):
            tol = 1e-2 if (half and nm in ("du", "ddelta", "dB", "dC")) else 1e-4
            e = relerr(a.float().cpu().numpy(), w_)
            assert e <= tol, (nm, e)


PACKED = [
    # Bt, Dm, H, W, N, K, Dd, dtype, kw: planes of at most 32 / 16 / 7 columns, two / four / eight to a wave
    (2, 24, 14, 14, 1, 4, None, torch.float32, {}),            # 6 channels per group: the second wave of a group holds two
    (2, 40, 7, 7, 2, 4, None, torch.bfloat16, {}),
    (3, 36, 9, 16, 4, 2, 18, torch.float32, {}),               # 16 columns exactly; delta shared by pairs of channels
    (2, 28, 20, 17, 1, 4, None, torch.float16, {}),            # two planes per wave, 7 channels per group
    (1, 64, 33, 32, 3, 4, 16, torch.float32, {}),              # 32 columns exactly, three states, delta shared by four channels
    (64, 96, 14, 14, 1, 4, None, torch.float32, {}),           # 6144 planes
    (2, 24, 15, 13, 1, 4, None, torch.float32, dict(dirs=capi.DIR_CORNERS, decay=0.9)),
    (2, 20, 10, 29, 2, 4, None, torch.float32, dict(dirs=capi.DIR_CORNERS, softplus=False)),
    (2, 24, 14, 14, 2, 4, None, torch.bfloat16, dict(out_float=False, use_D=False, use_bias=False)),
    (1, 4, 5, 1, 1, 1, None, torch.float32, {}),               # one column, one group
    # at most 7 columns: eight planes per wave
    (2, 72, 7, 7, 1, 4, None, torch.float32, {}),              # 18 channels per group
    (3, 36, 9, 6, 4, 2, 18, torch.float32, {}),                # delta shared by pairs of channels
    (3, 36, 9, 8, 4, 2, 18, torch.float32, {}),                # 8 columns: four planes per wave again
    (64, 384, 7, 7, 1, 4, None, torch.bfloat16, {}),
    (2, 40, 6, 5, 2, 4, None, torch.float16, {}),
    (2, 24, 7, 7, 1, 4, None, torch.float32, dict(dirs=capi.DIR_CORNERS, decay=0.9)),
    (2, 20, 10, 7, 3, 4, None, torch.float32, dict(dirs=capi.DIR_CORNERS, softplus=False)),
]


@pytest.mark.parametrize("Bt,Dm,H,W,N,K,Dd,dtype,kw", PACKED)
def test_wavefront_packed_planes(gpu_device, Bt, Dm, H, W, N, K, Dd, dtype, kw):
    """Several narrow planes per wave, forward and backward: against the tile kernels, and against the oracle where
    it takes the options."""
    print("wavefront packed planes", Bt, Dm, H, W, N, K, Dd, dtype, kw, flush=True)
    d, t, f, b = run(gpu_device, Bt, Dm, H, W, N, K, Dd, dtype, capi.SCHED_WAVEFRONT, **kw)
    _, _, f2, b2 = run(gpu_device, Bt, Dm, H, W, N, K, Dd, dtype, capi.SCHED_PLANE, **kw)
    half = dtype != torch.float32
    assert relerr(f.out.float().cpu().numpy(), f2.out.float().cpu().numpy()) <= (1e-2 if kw.get("out_float") is False else 1e-5)
    for nm, a, w_ in zip(NAMES, [b.du, b.ddelta, b.dA, b.dB, b.dC, b.dD, b.dbias, b.ddec], [b2.du, b2.ddelta, b2.dA, b2.dB, b2.dC, b2.dD, b2.dbias, b2.ddec]):
        assert (a is None) == (w_ is None), nm
        if a is None:
            continue
        tol = 1e-2 if (half and nm in ("du", "ddelta")) else (5e-4 if nm == "dA_decay" else 1e-4)
        e = relerr(a.float().cpu().numpy(), w_.float().cpu().numpy())
        assert e <= tol, (nm, e)
    check_against_oracle(d, t, f, b, Dd=Dd, **kw)   # and the float64 oracle under the same options


def test_packed_planes_keep_a_diverged_channel_inside_its_group(gpu_device):
    """Eight 7-column planes share a wave, separated by barrier lanes that stop the scan by a multiplication with
    zero: a channel that has run off to inf can therefore take the channel next to it in the wave along (inf * 0).
    All planes of a wave belong to one (batch, group) pair, whose dB / dC a diverged channel spoils in any case;
    pinned here: every other group comes out exactly as without the diverged channel."""
    Bt, Dm, H, W, N, K = 1, 16, 7, 7, 1, 2
    d = O.make_inputs(Bt, Dm, H, W, N=N, K=K, seed=21)
    res = {}
    for poisoned in (False, True):
        t = {k: torch.from_numpy(v).to(gpu_device) for k, v in d.items()}
        if poisoned:
            t["u"][0, 3, 2, 2] = float("inf")          # channel 3 of group 0 (channels 0-7)
        args = (t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"])
        f = capi.FwdCall(*args, True, True, None, True, capi.SCHED_WAVEFRONT)
        f.launch()
        b = capi.BwdCall(*args, t["dout"], f.x, f.x_v, True, None, f.x_sd, capi.SCHED_WAVEFRONT)
        b.launch()
        torch.cuda.synchronize()
        res[poisoned] = [x.clone() for x in (f.out, b.du, b.ddelta, b.dA, b.dB, b.dC, b.dD, b.dbias)]
    assert not torch.isfinite(res[True][0][0, 3]).all()            # the inf did reach channel 3's result
    rg = Dm // K
    for nm, clean, got in zip(["out"] + NAMES, res[False], res[True]):
        if nm in ("dB", "dC"):
            clean, got = clean[:, 1], got[:, 1]                     # [batch, group, ...]
        elif nm in ("out", "du", "ddelta"):
            clean, got = clean[:, rg:], got[:, rg:]
        else:
            clean, got = clean[rg:], got[rg:]
        assert torch.isfinite(got).all(), nm
        assert relerr(got.cpu().numpy(), clean.cpu().numpy()) <= 1e-6, nm


def _draw_large(seed):
    r = np.random.RandomState(7000 + seed)
    K = int(r.choice([2, 4]))
    rg = int(r.randint(33, 131))
    W = int(r.choice([r.randint(1, 8), r.randint(8, 17), r.randint(17, 33), r.randint(33, 65), r.randint(65, 257), r.randint(257, 513)]))
    Bt = int(r.choice([1, 2, 4]))
    if seed % 8 == 7:                                 # wide planes, more of them than CUs: blocks of 10 to 16 waves
        W, Bt = int(r.randint(257, 513)), 4
    return dict(Bt=Bt, K=K, Dm=K * rg, H=int(r.randint(1, 41)), W=W, N=int(r.choice([1, 2, 3, 4])),
                dtype=[torch.float32, torch.bfloat16, torch.float16][int(r.randint(3))], dirs=int(r.randint(2)),
                decay=0.9 if r.randint(4) == 0 else None)


@pytest.mark.parametrize("seed", range(32))
def test_wavefront_random_many_planes(gpu_device, seed):
    """Hundreds to thousands of planes of random size: every way the backward groups channels into blocks (one, two
    or four channels, two to eight planes per wave, blocks of up to 16 waves) with channel counts that leave ragged
    last blocks, against the tile kernels on the same inputs."""
    c = _draw_large(seed)
    print("wavefront random, many planes", seed, c, flush=True)
    kw = dict(dirs=c["dirs"], decay=c["decay"], seed=seed)
    d, t, f, b = run(gpu_device, c["Bt"], c["Dm"], c["H"], c["W"], c["N"], c["K"], None, c["dtype"], capi.SCHED_WAVEFRONT, **kw)
    _, _, f2, b2 = run(gpu_device, c["Bt"], c["Dm"], c["H"], c["W"], c["N"], c["K"], None, c["dtype"], capi.SCHED_PLANE, **kw)
    half = c["dtype"] != torch.float32
    assert relerr(f.out.cpu().numpy(), f2.out.cpu().numpy()) <= 1e-5
    for nm, a, w_ in zip(NAMES, [b.du, b.ddelta, b.dA, b.dB, b.dC, b.dD, b.dbias, b.ddec], [b2.du, b2.ddelta, b2.dA, b2.dB, b2.dC, b2.dD, b2.dbias, b2.ddec]):
        assert (a is None) == (w_ is None), nm
        if a is None:
            continue
        tol = 1e-2 if (half and nm in ("du", "ddelta")) else (5e-4 if nm == "dA_decay" else 1e-4)
        # (a single row or column makes some sums identically zero: both families then return rounding noise)
        ref = w_.float().cpu().numpy()
        scale = max(float(np.abs(ref).max()), 1e-6)
        e = float(np.abs(a.float().cpu().numpy().astype(np.float64) - ref).max()) / scale
        assert e <= tol or float(np.abs(ref).max()) < 1e-9, (nm, e)
    if seed % 4 == 0:                                 # a quarter of the sweep against the float64 oracle as well
        check_against_oracle(d, t, f, b, dirs=c["dirs"], decay=c["decay"])
