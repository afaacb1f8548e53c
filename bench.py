"""Benchmark of the 2D-CrossScan selective scan (selective_nd_scan fwd + bwd) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c1|c2|c3|c4|c4n1|c1n1|c2n1] [--no-cpu]

One step = one forward + one backward of the operator through the PyTorch extension (output,
saved-state and gradient allocations, zero-fills and dtype casts included, as a caller of the
reference's fwd/bwd bindings would pay them) on synthetic inputs already resident in HBM.
Prints ONE JSON line.  `value` is the algorithmic HBM rate of the whole step:
    bytes = (2eP + 2eQ + 4P) + (4eP + 4eQ + 4P),  P = B*D*H*W, Q = B*K*N*H*W, e = input bytes
(compulsory tensor I/O only) divided by the mean step time.  `roofline` is the same figure for the
dominant kernel alone (the backward), from one pair of HIP events on the launch stream around K back-to-back
launches of it through the C ABI (after W untimed ones; defaults K = 50, W = 20: the clocks settle over the first
10-15 steps after the host-side input generation), with a second leg beside it: vector-ALU wave-instructions per
second against the published FP32 vector peak (157.3 TFLOP/s = 1228.9 G wave-wide multiply-adds per second), with
the rate a pure multiply-add stream reaches on all CUs beside it (`valu.probe_peak`, from
profiles/issue_probe_mi355x.txt).  `roofline_fwd` is the same pair of figures for the forward kernel, plus the
rate of its real memory traffic (checkpoints and re-reads included).  The instruction count, the clock and the
traffic per launch are counter readings that a timed run cannot take; they come from the committed rocprofv3
summary of the same workload under profiles/ (named in `counters_from`) and are used only if that summary was
taken from the kernel sources of this tree (`kernel_source_sha`) and its kernel durations agree with the ones
measured here within 5 % (4 µs for the shortest kernels; `profile_vs_live`); otherwise they are left out (null) and `counters_stale` says why.
Every duration is measured live.  `roofline.bound` names the leg with the higher fraction.
`cpu_baseline` times the C restatement of the reference recurrence (oracle/) on the host cores on a bounded sample
of the same workload; `cpu_baseline_torch` the line-for-line PyTorch transcription of the recurrence (forward, and
autograd through it for the backward) on a smaller sample.
"""
import argparse
import json
import math
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "official-cross-scan_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

METRIC = "fwd+bwd 2D-scan ms/iter & HBM GB/s (% peak), "     # + the workload: B64 D192 56x56 N16 K4 for c1
HBM_PEAK_GBS = 8000.0           # MI355X HBM3E, published peak
WORKLOADS = {                   # name: (B, D, H, W, N, K, input dtype)
    "c1": (64, 192, 56, 56, 16, 4, "float32"),
    "c2": (64, 768, 14, 14, 16, 4, "bfloat16"),
    "c3": (2, 192, 200, 336, 16, 4, "float32"),
    "c4": (1, 256, 512, 512, 16, 4, "bfloat16"),
    "c4n1": (1, 256, 512, 512, 1, 4, "bfloat16"),
    "c1n1": (64, 192, 56, 56, 1, 4, "float32"),     # c1's planes with one state per channel (the d_state = 1 variant)
    "c2n1": (64, 768, 14, 14, 1, 4, "bfloat16"),    # c2's planes with one state per channel
}


def algorithmic_bytes(Bt, Dm, H, W, N, K, e):
    P, Q = Bt * Dm * H * W, Bt * K * N * H * W
    return 2 * e * P + 2 * e * Q + 4 * P, 4 * e * P + 4 * e * Q + 4 * P


def make_inputs(torch, Bt, Dm, H, W, N, K, dtype, dev):
    """Value distributions of the headline metric, generated on the device, seed 0."""
    g = torch.Generator(device=dev)
    g.manual_seed(0)
    rn = lambda *s: torch.randn(*s, device=dev, generator=g)
    u = rn(Bt, Dm, H, W).to(dtype)
    delta = (0.1 * rn(Bt, Dm, H, W)).to(dtype)
    dt = torch.exp(torch.empty(Dm, device=dev).uniform_(math.log(1e-3), math.log(1e-1), generator=g))
    bias = torch.log(torch.expm1(dt))
    A = -torch.arange(1, N + 1, device=dev, dtype=torch.float32).repeat(Dm, 1).contiguous()
    B = rn(Bt, K, N, H, W).to(dtype)
    C = rn(Bt, K, N, H, W).to(dtype)
    D = torch.ones(Dm, device=dev)
    dout = rn(Bt, Dm, H, W)
    return u, delta, A, B, C, D, bias, dout


def cpu_baseline(workload, budget_s=20.0):
    """C restatement of the reference recurrence (fp32 state) on the host cores, fwd + bwd, on a
    slice of the batch, repeated until roughly `budget_s` core-seconds of CPU work are spent."""
    import numpy as np
    from oracle import snd_oracle as O
    from oracle import snd_oracle_c as OC
    Bt, Dm, H, W, N, K, dtn = WORKLOADS[workload]
    env = os.environ.get("OMP_NUM_THREADS", "")
    cores = int(env) if env.isdigit() and int(env) > 0 else (os.cpu_count() or 1)

    def run(sb, sd):
        d = O.make_inputs(sb, sd, H, W, N=N, K=K, seed=0)
        a = (d["u"], d["delta"], d["A"], d["B"], d["C"], d["D"], d["delta_bias"])
        t0 = time.perf_counter()
        OC.fwd(*a, True, None, nthreads=cores)
        OC.bwd(*a, d["dout"], True, None, nthreads=cores)
        return time.perf_counter() - t0

    # planes are independent, so a slice of the batch (of the channels when B == 1) is the same work
    # per element; grow the slice until one fwd+bwd takes about budget_s of wall time
    if Bt > 1:
        sb, sd = min(Bt, max(1, (cores + K - 1) // K)), Dm
    else:
        sb, sd = 1, min(Dm, K * max(1, cores // K))
    t = run(sb, sd)
    if t * cores < 0.5 * budget_s:
        grow = budget_s / max(t * cores, 1e-6)
        if Bt > 1:
            sb = int(max(sb, min(Bt, sb * grow)))
        else:
            sd = int(max(sd, min(Dm, (int(sd * grow) // K) * K)))
    # repeat the slice until about budget_s core-seconds of CPU work are spent; report the mean
    times = []
    while not times or sum(times) * cores < budget_s:
        times.append(run(sb, sd))
    t = sum(times) / len(times)
    fb, bb = algorithmic_bytes(sb, sd, H, W, N, K, 4)
    return {"value": round((fb + bb) / t / 1e9, 4), "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": "%s slice B=%d D=%d (fp32 I/O, fp32 state), fwd+bwd x%d, %.2f s wall each (%.0f core-seconds in all), %.3f ms per (b,c) plane set"
                      % (workload, sb, sd, len(times), t, sum(times) * cores, 1e3 * t / (sb * sd)),
            "ms_per_step_extrapolated": round(1e3 * t * (Bt * Dm) / (sb * sd), 1)}


VALU_PEAK = 157.3e12 / 128.0    # published FP32 vector peak in wave-wide multiply-adds per second (64 lanes x 2 flop)


def probe_peak():
    """Wave-instructions per second of a pure v_fma_f32 stream on all CUs, from the committed summary of the
    instruction-issue micro-benchmark, or None."""
    path = os.path.join(ROOT, "profiles", "issue_probe_mi355x.txt")
    if not os.path.exists(path):
        return None
    m = re.search(r"^fma_stream_ginst_per_s:\s*([0-9.]+)", open(path).read(), flags=re.M)
    return float(m.group(1)) * 1e9 if m else None


def kernel_source_sha():
    """sha256 (16 hex digits) over the kernel sources (csrc/*.h, *.hip, in name order): stored in every profile summary
    under profiles/ and compared here, so that counters taken from other kernels than the ones that run are not used."""
    import glob
    import hashlib
    h = hashlib.sha256()
    csrc = os.path.join(ROOT, "official-cross-scan_amd", "csrc")
    for path in sorted(glob.glob(os.path.join(csrc, "*.h")) + glob.glob(os.path.join(csrc, "*.hip"))):
        h.update(os.path.basename(path).encode() + b"\0" + open(path, "rb").read())
    return h.hexdigest()[:16]


def profile_counters(workload):
    """Counter readings of the two kernels from the committed rocprofv3 summary of this workload: kernel names, memory
    traffic per launch, VALU wave-instructions per launch, shader clock under this load, average durations, and the
    hash of the kernel sources the summary was taken from.  A timed run cannot read counters; durations are always
    measured live."""
    rel = os.path.join("profiles", "bwd_kernel_%s_pmc.txt" % workload)
    path = os.path.join(ROOT, rel)
    if not os.path.exists(path):
        return None
    text = open(path).read()
    out = {"file": rel}
    for key in ("dominant_kernel", "avg_ns", "traffic_bytes_per_launch", "valu_insts_per_launch", "clock_ghz",
                "fwd_kernel", "fwd_avg_ns", "fwd_traffic_bytes_per_launch", "fwd_valu_insts_per_launch", "fwd_clock_ghz",
                "kernel_source_sha"):
        m = re.search(r"^%s:\s*(.+)$" % key, text, flags=re.M)
        if not m:
            if key == "kernel_source_sha":
                out[key] = None
                continue
            return None
        out[key] = m.group(1).strip() if key in ("dominant_kernel", "fwd_kernel", "kernel_source_sha") else float(m.group(1))
    return out


def cpu_baseline_torch(workload, budget_s=12.0):
    """The line-for-line PyTorch transcription of the reference recurrence (oracle/snd_torch_ref.py: a row loop over a
    column loop of h = a*(h_left + h_up - 0.5*(a_up + a_left)*h_diag) + bu, vectorised over (batch, channel, state)),
    forward and autograd backward, fp32, on the host cores, on a slice of the workload sized to a few seconds."""
    import torch
    from oracle import snd_oracle as O
    from oracle.snd_torch_ref import selective_nd_scan_torch
    Bt, Dm, H, W, N, K, dtn = WORKLOADS[workload]
    env = os.environ.get("OMP_NUM_THREADS", "")
    cores = int(env) if env.isdigit() and int(env) > 0 else (os.cpu_count() or 1)
    torch.set_num_threads(cores)
    # the python loops cost about a millisecond per cell (forward + backward) whatever the slice holds, so the slice is
    # 3072 (channel, state) planes wide (autograd keeps a dozen fp32 values per state-cell: ~150 KB per cell) and as
    # many rows long as the budget allows: the first rows of the plane, all of them where they fit
    rows = max(4, min(H, int(budget_s / 1e-3) // W))
    sd = min(Dm, K * max(1, 3072 // (K * N)))
    d = O.make_inputs(1, sd, rows, W, N=N, K=K, seed=0)
    t = {k: torch.from_numpy(v) for k, v in d.items()}
    leaves = [t[k].clone().requires_grad_(True) for k in ("u", "delta", "A", "B", "C", "D", "delta_bias")]
    t0 = time.perf_counter()
    out = selective_nd_scan_torch(*leaves, delta_softplus=True)
    t1 = time.perf_counter()
    out.backward(t["dout"])
    t2 = time.perf_counter()
    fb, bb = algorithmic_bytes(1, sd, rows, W, N, K, 4)
    full = (t2 - t0) * (Bt * Dm * H) / (sd * rows)
    return {"value": round((fb + bb) / (t2 - t0) / 1e9, 5), "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": "%s slice B=1 D=%d rows=%d of %d (fp32), forward %.2f s + autograd backward %.2f s, once"
                      % (workload, sd, rows, H, t1 - t0, t2 - t1),
            "ms_per_step_extrapolated": round(1e3 * full, 0)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # (the clocks settle over the first 10-15 steps after the seconds of host-side input generation: c1 takes 2.25 ms
    # for its second step and 1.89 ms from the fourteenth on; the warm-up covers that)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c1", choices=sorted(WORKLOADS))
    ap.add_argument("--shape", default=None, metavar="B,D,H,W,N,K,dtype",
                    help="time another shape than the named workloads (same value distributions), e.g. 64,192,56,56,5,4,float32; "
                         "no committed counters exist for such a shape, so the roofline objects carry the timed legs only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the host-CPU baseline leg")
    ap.add_argument("--schedule", default="auto", choices=["auto", "plane", "strips", "bands", "wavefront"],
                    help="kernel family and block mapping: chosen by shape (default), one block per plane chunk, "
                         "pipelined row strips / bands, or the row-segment wavefront kernels (1-4 states)")
    ap.add_argument("--strip-segments", type=int, default=0, metavar="N",
                    help="timing studies: force the column segments per strip of the pipelined 16-state backward "
                         "(1 = whole strips; 0 = the library's own choice)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this operator is measured on ONE GPU (every (batch, channel, state) plane is an "
                 "independent recurrence; multi-GPU is plain batch sharding and is not part of this build). "
                 "Run with --gpus 1.")

    import torch
    dev = torch.device("cuda:0")
    import selective_nd_scan as snd
    from selective_nd_scan import capi

    sched = {"auto": 0, "plane": 1, "strips": 2, "bands": 3, "wavefront": 4}[args.schedule]
    snd.set_schedule(sched)
    if args.strip_segments:
        capi.lib().snd_debug_set_strip_slots(-args.strip_segments)
    if args.shape:
        f_ = args.shape.split(",")
        WORKLOADS["custom"] = tuple(int(v) for v in f_[:6]) + (f_[6],)
        args.workload = "custom"
    Bt, Dm, H, W, N, K, dtn = WORKLOADS[args.workload]
    dtype = getattr(torch, dtn)
    u, delta, A, B, C, D, bias, dout = make_inputs(torch, Bt, Dm, H, W, N, K, dtype, dev)
    fb, bb = algorithmic_bytes(Bt, Dm, H, W, N, K, u.element_size())

    def step():
        out, x, x_v, x_sd = snd.fwd(u, delta, A, B, C, D, bias, True, True, None)
        return snd.bwd(u, delta, A, B, C, D, bias, dout, x, x_v, True, None, x_sd)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps

    # kernel-only durations: HIP events on the launch stream around launches through the C ABI
    fcall = capi.FwdCall(u, delta, A, B, C, D, bias, True, True, None, True, sched)
    fcall.launch()
    bcall = capi.BwdCall(u, delta, A, B, C, D, bias, dout, fcall.x, fcall.x_v, True, None, fcall.x_sd, sched)
    stream = torch.cuda.current_stream()
    # (each kernel launched back to back between ONE pair of events and divided by the count: a pair of events around
    # every launch would add the event and launch gaps, a few microseconds, to every figure)
    def kernel_ms(launch):
        for _ in range(args.warmup):
            launch()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(args.steps):
            launch()
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.steps
    kf_ms = kernel_ms(fcall.launch)
    bcall.zero()
    kb_ms = kernel_ms(bcall.launch_kernel_only)     # (the accumulated gradients are not cleared in between: timing only)

    value = (fb + bb) / (ms * 1e-3) / 1e9
    st, plan = capi.make_plan(capi.make_shape(u, delta, A, B))
    capi.check(st)
    used = sched if sched else plan.auto_schedule
    wave = used == capi.SCHED_WAVEFRONT
    pp = probe_peak()

    def leg(kernel, alg_bytes, k_ms):
        ach = alg_bytes / (k_ms * 1e-3) / 1e9
        return {"bound": "hbm", "kernel": kernel, "achieved": round(ach, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(ach / HBM_PEAK_GBS, 4), "traffic": None, "algorithmic_bytes_per_launch": alg_bytes,
                "kernel_ms": round(k_ms, 4)}

    def add_counters(r, k_ms, file, traffic, insts, clock, prof_ns):
        rate = insts / (k_ms * 1e-3)
        r.update({"traffic": traffic, "traffic_GBs": round(traffic / (k_ms * 1e-3) / 1e9, 1), "counters_from": file,
                  "profile_kernel_ms": round(prof_ns * 1e-6, 4), "profile_vs_live": round(prof_ns * 1e-6 / k_ms, 3),
                  "valu": {"insts_per_launch": insts, "clock_ghz": clock, "achieved": round(rate / 1e9, 2),
                           "peak": round(VALU_PEAK / 1e9, 2), "probe_peak": round(pp / 1e9, 2) if pp else None,
                           "unit": "G wave-instructions/s"},
                  "frac_valu": round(rate / VALU_PEAK, 4)})
        if r["frac_valu"] > r["frac"]:
            r["bound"] = "valu"

    roof = leg("snd::wave_bwd_kernel" if wave else "snd::bwd_kernel", bb, kb_ms)
    roof_fwd = leg("snd::wave_fwd_kernel" if wave else "snd::fwd_kernel", fb, kf_ms)
    pc = profile_counters(args.workload) if args.schedule == "auto" and not args.shape else None
    if pc:
        # counters from the committed profile of this workload, if it is a profile of these kernels: same kernel,
        # same sources, and durations that agree with the ones measured here
        stale = None
        if not pc["dominant_kernel"].startswith(roof["kernel"] + "<") or not pc["fwd_kernel"].startswith(roof_fwd["kernel"] + "<"):
            stale = "the profile is of other kernels (%s)" % pc["dominant_kernel"].split("<")[0]
        elif pc["kernel_source_sha"] != kernel_source_sha():
            stale = "the profile was taken from other kernel sources (%s, here %s)" % (pc["kernel_source_sha"], kernel_source_sha())
        # (within 5 %, or within 4 microseconds for kernels of a few tens of microseconds: the durations measured here are
        # K back-to-back launches between two events and include the gap between launches, the profile's do not)
        elif not (abs(pc["avg_ns"] * 1e-6 - kb_ms) <= max(0.05 * kb_ms, 0.004) and abs(pc["fwd_avg_ns"] * 1e-6 - kf_ms) <= max(0.05 * kf_ms, 0.004)):
            stale = "kernel durations differ from the profile's by more than 5 %% (bwd %.3f, fwd %.3f)" % (
                pc["avg_ns"] * 1e-6 / kb_ms, pc["fwd_avg_ns"] * 1e-6 / kf_ms)
        if stale is None:
            add_counters(roof, kb_ms, pc["file"], pc["traffic_bytes_per_launch"], pc["valu_insts_per_launch"], pc["clock_ghz"], pc["avg_ns"])
            add_counters(roof_fwd, kf_ms, pc["file"], pc["fwd_traffic_bytes_per_launch"], pc["fwd_valu_insts_per_launch"],
                         pc["fwd_clock_ghz"], pc["fwd_avg_ns"])
        else:
            roof["counters_stale"] = roof_fwd["counters_stale"] = "%s: %s" % (pc["file"], stale)
    rec = {
        "metric": METRIC + "B%d D%d %dx%d N%d K%d" % (Bt, Dm, H, W, N, K), "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak",
        # arithmetic type of the recurrence and of every accumulation, whatever the I/O dtype of the workload
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "%s: selective_nd_scan fwd+bwd, B=%d D=%d H=%d W=%d N=%d K=%d, %s inputs, fp32 state"
                               % (args.workload, Bt, Dm, H, W, N, K, dtn),
                   "io_dtype": dtn, "schedule": args.schedule, "algorithmic_bytes": fb + bb, "pct_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
                   "pixels_per_s": round(Bt * Dm * H * W / (ms * 1e-3), 1),
                   "state_cells_per_s": round(Bt * Dm * H * W * N / (ms * 1e-3), 1),
                   "kernel_ms": {"fwd": round(kf_ms, 4), "bwd": round(kb_ms, 4)},
                   "kernel_only_GBs": round((fb + bb) / ((kf_ms + kb_ms) * 1e-3) / 1e9, 2)},
        "roofline": roof,
        "roofline_fwd": roof_fwd,
    }
    if not args.no_cpu:
        rec["cpu_baseline"] = cpu_baseline(args.workload)
        rec["cpu_baseline_torch"] = cpu_baseline_torch(args.workload)
    print(json.dumps(rec))


if __name__ == "__main__":
    main()
