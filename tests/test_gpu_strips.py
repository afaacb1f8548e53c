"""Pipelined schedules (one block per 8-row strip, or per band of strips in the backward; jobs drawn
from ticket queues, hand-over through per-strip progress counts) against the whole-plane schedule and
the oracle."""
import numpy as np
import pytest
import torch

import capi
from oracle import snd_oracle as O
from oracle import snd_oracle_c as OC
from test_gpu_fwd import relerr

pytestmark = pytest.mark.gpu
NAMES = ["du", "ddelta", "dA", "dB", "dC", "dD", "ddelta_bias"]

SHAPES = [
    # Bt, Dm, H, W, N, K, dtype
    (2, 16, 56, 56, 16, 4, torch.float32),     # 7 strips x 7 tiles
    (1, 8, 17, 9, 16, 2, torch.float32),       # ragged edges, 3 strips x 2 tiles
    (1, 32, 64, 8, 16, 1, torch.float32),      # one column tile: the row hand-over is the only carry
    (1, 4, 24, 40, 4, 2, torch.float32),       # 8-state kernels
    (1, 8, 100, 70, 16, 4, torch.bfloat16),
    (3, 20, 33, 21, 5, 1, torch.float16),      # partial channel chunk (20 = 16 + 4), odd N
    (1, 8, 35, 21, 16, 2, torch.float32),      # 7x7 tiles: 5 strips x 3 tiles
    (2, 16, 27, 14, 8, 4, torch.bfloat16),     # 7x7 tiles, ragged last strip, 8-state kernels
    (8, 32, 40, 24, 16, 4, torch.float32),     # 32 (batch, group) pairs: one job queue per XCD, 4 pairs each
    (5, 64, 30, 17, 8, 4, torch.bfloat16),     # 20 pairs: queues of 3 and 2 pairs (uneven: blocks take from other queues)
    (4, 96, 23, 9, 16, 4, torch.float32),      # 16 pairs x 2 channel chunks (24 = 16 + 8), 3 strips
]


def sync_error(ws):
    return int(ws.view(torch.int32)[1].item())


@pytest.mark.parametrize("Bt,Dm,H,W,N,K,dtype", SHAPES)
def test_strips_match_plane_and_oracle(gpu_device, Bt, Dm, H, W, N, K, dtype):
    print("strips", Bt, Dm, H, W, N, K, dtype, flush=True)
    d = O.make_inputs(Bt, Dm, H, W, N=N, K=K, seed=5)
    t = {k: torch.from_numpy(v).to(gpu_device) for k, v in d.items()}
    for k in ("u", "delta", "B", "C"):
        t[k] = t[k].to(dtype)
    args = (t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"])
    res = {}
    for sched in (capi.SCHED_PLANE, capi.SCHED_STRIPS, capi.SCHED_BANDS):
        f = capi.FwdCall(*args, True, True, None, True, sched)
        f.ws.view(torch.int32)[:16] = 0x7fffffff              # the library must clear its sync words itself
        f.launch()
        b = capi.BwdCall(*args, t["dout"], f.x, f.x_v, True, None, f.x_sd, sched)
        b.ws.view(torch.int32)[:16] = 0x7fffffff
        b.launch()
        torch.cuda.synchronize()
        if sched != capi.SCHED_PLANE:
            assert sync_error(f.ws) == 0 and sync_error(b.ws) == 0, "a strip wait ran into its poll limit"
        res[sched] = (f.out, [b.du, b.ddelta, b.dA, b.dB, b.dC, b.dD, b.dbias], (f.x, f.x_v, f.x_sd))
    out_p, g_p, st_p = res[capi.SCHED_PLANE]
    out_s, g_s, st_s = res[capi.SCHED_STRIPS]
    ncx = f.plan.n_chunks_x
    for sched in (capi.SCHED_STRIPS, capi.SCHED_BANDS):
        out_q, g_q, st_q = res[sched]
        # same arithmetic in the same order per plane: everything that is not an atomic sum is bit-identical
        assert torch.equal(out_p, out_q)
        used_v = Bt * f.plan.n_chunks_y * ncx * 8 * Dm * N
        assert torch.equal(st_p[1].reshape(-1)[:used_v], st_q[1].reshape(-1)[:used_v])   # x_v: every entry of the tile layout is written
        used = Bt * ncx * f.plan.n_chunks_y * 8 * Dm * N          # what the tile layout occupies (the buffers may be larger)
        for a, b_ in ((st_p[0], st_q[0]), (st_p[2], st_q[2])):    # x, x_sd: stored tile-major, last column tile unused
            assert torch.equal(a.reshape(-1)[:used].reshape(Bt, ncx, -1)[:, :ncx - 1], b_.reshape(-1)[:used].reshape(Bt, ncx, -1)[:, :ncx - 1])
        assert torch.equal(g_p[0], g_q[0]) and torch.equal(g_p[1], g_q[1])
        for nm, a, b_ in zip(NAMES[2:], g_p[2:], g_q[2:]):        # atomic sums: same terms, other order
            assert relerr(a.float().cpu().numpy(), b_.float().cpu().numpy()) <= 1e-5, (sched, nm)
    r = {k: t[k].float().cpu().numpy() for k in ("u", "delta", "B", "C")}
    ref = OC.fwd(r["u"], r["delta"], d["A"], r["B"], r["C"], d["D"], d["delta_bias"], True, None, real="f64")
    gref = OC.bwd(r["u"], r["delta"], d["A"], r["B"], r["C"], d["D"], d["delta_bias"], d["dout"], True, None, real="f64")
    assert relerr(out_s.cpu().numpy(), ref) <= 1e-4
    half = dtype != torch.float32
    for nm, a, b_ in zip(NAMES, g_s, gref):
        tol = 1e-2 if (half and nm in ("du", "ddelta", "dB", "dC")) else 1e-4
        assert relerr(a.float().cpu().numpy(), b_) <= tol, (nm, relerr(a.float().cpu().numpy(), b_))


def test_strips_inference_only(gpu_device):
    """x = x_sd = null (no column checkpoints) with the strip schedule."""
    d = O.make_inputs(1, 16, 40, 24, N=16, K=2, seed=9)
    t = {k: torch.from_numpy(v).to(gpu_device) for k, v in d.items()}
    args = (t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"])
    f = capi.FwdCall(*args, True, True, None, False, capi.SCHED_STRIPS)
    f.launch()
    torch.cuda.synchronize()
    assert sync_error(f.ws) == 0
    ref = OC.fwd(d["u"], d["delta"], d["A"], d["B"], d["C"], d["D"], d["delta_bias"], True, None, real="f64")
    assert relerr(f.out.cpu().numpy(), ref) <= 1e-4


def test_strips_need_workspace(gpu_device):
    d = O.make_inputs(1, 4, 16, 16, N=4, K=1, seed=1)
    t = {k: torch.from_numpy(v).to(gpu_device) for k, v in d.items()}
    f = capi.FwdCall(t["u"], t["delta"], t["A"], t["B"], t["C"], None, None, False, True, None, True, capi.SCHED_STRIPS)
    f.params.workspace = None
    assert capi.lib().snd_fwd(capi.C.byref(f.params), torch.cuda.current_stream().cuda_stream) == -6
    f.params.workspace, f.params.workspace_bytes = f.ws.data_ptr(), 8
    assert capi.lib().snd_fwd(capi.C.byref(f.params), torch.cuda.current_stream().cuda_stream) == -6


@pytest.mark.parametrize("Bt,Dm,H,W,N,K,dtype,slots", [
    (1, 32, 100, 70, 16, 4, torch.float32, -2),       # 4 plane chunks x 13 strips x 9 tiles, two segments (4 + 5 tiles)
    (2, 48, 61, 131, 16, 2, torch.float32, -3),       # ragged strips and tiles, partial channel chunks (24 = 16 + 8), 17 tiles in three segments
    (1, 16, 200, 96, 12, 1, torch.bfloat16, -4),      # one plane chunk, 25 strips x 12 tiles, vector staging of 16-bit inputs
    (1, 64, 90, 133, 16, 4, torch.float16, -2),       # unaligned rows (element-wise staging)
    (1, 8, 40, 21, 16, 2, torch.float32, -8),         # 7x7 tiles, three tiles: one segment of two tiles is all that fits
])
def test_column_segmented_strips(gpu_device, Bt, Dm, H, W, N, K, dtype, slots):
    """The backward's strips cut into column segments (taken where there are more strip jobs than block slots; here
    forced through the test hook): bit-identical du / ddelta to whole strips and to whole planes, sums to
    rounding, everything against the float64 oracle."""
    print("column segments", Bt, Dm, H, W, N, K, dtype, slots, flush=True)
    lib = capi.lib()
    d = O.make_inputs(Bt, Dm, H, W, N=N, K=K, seed=21)
    t = {k: torch.from_numpy(v).to(gpu_device) for k, v in d.items()}
    for k in ("u", "delta", "B", "C"):
        t[k] = t[k].to(dtype)
    args = (t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"])
    f = capi.FwdCall(*args, True, True, None, True, capi.SCHED_PLANE)
    f.launch()
    res = {}
    try:
        for name, sched, sl in (("plane", capi.SCHED_PLANE, 0), ("strips", capi.SCHED_STRIPS, 0), ("segments", capi.SCHED_STRIPS, slots)):
            lib.snd_debug_set_strip_slots(sl)
            b = capi.BwdCall(*args, t["dout"], f.x, f.x_v, True, None, f.x_sd, sched)
            if name == "segments":
                st, plan = capi.make_plan(capi.make_shape(t["u"], t["delta"], t["A"], t["B"]))
                assert (plan.bwd_workspace_bytes > plan.fwd_workspace_bytes) == (plan.n_chunks_x >= 4), "this shape was meant to take column segments"
            b.ws.view(torch.int32)[:16] = 0x7fffffff
            b.launch()
            torch.cuda.synchronize()
            if sched != capi.SCHED_PLANE:
                assert sync_error(b.ws) == 0, "a wait ran into its poll limit"
            res[name] = [b.du, b.ddelta, b.dA, b.dB, b.dC, b.dD, b.dbias]
    finally:
        lib.snd_debug_set_strip_slots(0)
    for name in ("strips", "segments"):
        assert torch.equal(res["plane"][0], res[name][0]) and torch.equal(res["plane"][1], res[name][1]), name
        for nm, a, b_ in zip(NAMES[2:], res["plane"][2:], res[name][2:]):
            assert relerr(a.float().cpu().numpy(), b_.float().cpu().numpy()) <= 1e-5, (name, nm)
    r = {k: t[k].float().cpu().numpy() for k in ("u", "delta", "B", "C")}
    gref = OC.bwd(r["u"], r["delta"], d["A"], r["B"], r["C"], d["D"], d["delta_bias"], d["dout"], True, None, real="f64")
    half = dtype != torch.float32
    for nm, a, b_ in zip(NAMES, res["segments"], gref):
        tol = 1e-2 if (half and nm in ("du", "ddelta", "dB", "dC")) else 1e-4
        assert relerr(a.float().cpu().numpy(), b_) <= tol, (nm, relerr(a.float().cpu().numpy(), b_))
