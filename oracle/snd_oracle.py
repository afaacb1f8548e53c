"""CPU oracle for the 2D-CrossScan selective scan (forward + hand adjoint), float64 numpy.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this module; it is the
checker used by tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py.

It restates, cell by cell, what the reference CUDA kernels compute:

* forward  : kernels/selective_nd_scan/include/cusoflex/selective_scan_fwd_kernel_oflex.cuh:189-346
             (delta bias + softplus :221-224, a = exp2(delta*A*log2e)*A_decay :194-195,245,
              neighbour recurrence :263-272 + row scan :289-292, "SD" row-only branch :306-337,
              output accumulation :226-228,301,334; defaults D=0, bias=0, A_decay=1 :121-134)
* scan op  : kernels/selective_nd_scan/include/selective_scan_common.h:100-107
             ((a0,b0) o (a1,b1) = (a1*a0, a1*b0+b1), i.e. h_j = a_j*h_{j-1} + b_j)
* constants: selective_scan_common.h:13-21 (WEIGHT_LT_H 0.5, WEIGHT_DELTA_A_EXP 1.0, SD_SWITCH_ON 1),
             0.25 self-term weight fwd.cuh:334, softplus threshold 20 fwd.cuh:223
* backward : kernels/selective_nd_scan/include/cusoflex/selective_scan_bwd_kernel_oflex.cuh
             :207-214 (D*dout, dD), :383-612 (adjoint recurrence and gradients of the main branch),
             :621-775 (SD branch), :785-819 (softplus gradient, ddelta_bias)
* host post-processing: kernels/selective_nd_scan/src/cusoflex/selective_scan_oflex.cpp:250
             (out dtype), :393-403 (gradient dtypes), :432-438 (group sums of ddelta / ddelta_bias)

Pinning (see tests/test_oracle_pins.py): H=1 / W=1 reductions to the textbook 1D selective scan,
constant-a separable geometric closed form, a=f(i+j) closed form, transpose symmetry, linearity in
u, an anti-diagonal-order re-evaluation, explicit impulse responses on tiny grids, and for the
adjoint torch.autograd (float64) through an independent torch restatement plus finite differences.
The reference ships no tests or golden vectors for this path, so these are what pin it.

Known, deliberate difference from the reference: dA_decay here is the true gradient (includes
the SD branch); the reference's omits the SD-branch term (bwd.cuh:746-756 has no dA_decay line).
"""
import numpy as np

WEIGHT_LT_H = 0.5          # selective_scan_common.h:20
WEIGHT_SELF = 0.25         # fwd.cuh:334
SOFTPLUS_THRESHOLD = 20.0  # fwd.cuh:223


def _prep(u, delta, A, B, C, D, delta_bias, delta_softplus, A_decay):
    """Expand everything to per-channel float64 arrays.  Shapes follow host.cpp:206-229."""
    u = np.asarray(u, dtype=np.float64)
    delta = np.asarray(delta, dtype=np.float64)
    A = np.asarray(A, dtype=np.float64)
    B = np.asarray(B, dtype=np.float64)
    C = np.asarray(C, dtype=np.float64)
    Bt, Dm, H, W = u.shape
    Dd = delta.shape[1]
    G = B.shape[1]
    N = A.shape[1]
    assert Dm % G == 0 and Dm % Dd == 0
    assert delta.shape == (Bt, Dd, H, W) and A.shape == (Dm, N)
    assert B.shape == (Bt, G, N, H, W) and C.shape == (Bt, G, N, H, W)
    rd = Dm // Dd
    rg = Dm // G
    raw = np.repeat(delta, rd, axis=1)                                   # fwd.cuh:106,109
    if delta_bias is not None:
        raw = raw + np.repeat(np.asarray(delta_bias, np.float64), rd)[None, :, None, None]
    if delta_softplus:                                                   # fwd.cuh:222-224
        with np.errstate(over="ignore"):
            dl = np.where(raw <= SOFTPLUS_THRESHOLD, np.log1p(np.exp(np.minimum(raw, 50.0))), raw)
    else:
        dl = raw
    adec = 1.0 if A_decay is None else float(np.asarray(A_decay, np.float64).reshape(-1)[0])
    a = np.exp(dl[:, :, None] * A[None, :, :, None, None]) * adec        # fwd.cuh:194-195,245
    Bc = np.repeat(B, rg, axis=1)                                        # fwd.cuh:105,112
    Cc = np.repeat(C, rg, axis=1)
    bu = Bc * (dl * u)[:, :, None]                                       # fwd.cuh:225,265
    Dv = np.zeros(Dm) if D is None else np.asarray(D, np.float64)        # fwd.cuh:121-124
    return u, raw, dl, A, Bc, Cc, a, bu, Dv, adec, (Bt, Dm, H, W, Dd, G, N, rd, rg)


def scan_states(a, bu, sd=True):
    """h (2D neighbour recurrence) and s (row-only scan) for arrays [..., H, W]."""
    H, W = a.shape[-2:]
    h = np.zeros_like(bu)
    s = np.zeros_like(bu)
    zero = np.zeros(a.shape[:-2])
    for i in range(H):
        for j in range(W):
            left = h[..., i, j - 1] if j > 0 else zero
            up = h[..., i - 1, j] if i > 0 else zero
            if i > 0 and j > 0:
                diag = h[..., i - 1, j - 1]
                corr = WEIGHT_LT_H * (a[..., i - 1, j] + a[..., i, j - 1]) * diag   # fwd.cuh:265,270
            else:
                corr = zero
            h[..., i, j] = a[..., i, j] * (left + up - corr) + bu[..., i, j]        # fwd.cuh:263-272,290
            if sd:
                sl = s[..., i, j - 1] if j > 0 else zero
                s[..., i, j] = a[..., i, j] * sl + bu[..., i, j]                    # fwd.cuh:309-327
    return h, s


def selective_nd_scan_fwd(u, delta, A, B, C, D=None, delta_bias=None, delta_softplus=False,
                          A_decay=None, sd=True, return_states=False):
    """out[b,c,i,j] = D*u + sum_n C*(h - s + 0.25*bu)   (sd=True, the shipped SD_SWITCH_ON=1 build)
                    = D*u + sum_n C*h                    (sd=False)."""
    u, raw, dl, A, Bc, Cc, a, bu, Dv, adec, dims = _prep(u, delta, A, B, C, D, delta_bias,
                                                        delta_softplus, A_decay)
    h, s = scan_states(a, bu, sd)
    y = h - s + WEIGHT_SELF * bu if sd else h                            # fwd.cuh:301,334
    out = Dv[None, :, None, None] * u + (Cc * y).sum(axis=2)             # fwd.cuh:227
    if return_states:
        return out, h, s
    return out


def _shift(x, di, dj):
    """y[..., i, j] = x[..., i+di, j+dj] with zeros outside the plane."""
    H, W = x.shape[-2:]
    y = np.zeros_like(x)
    si = slice(max(0, -di), H - max(0, di))
    sj = slice(max(0, -dj), W - max(0, dj))
    ti = slice(max(0, di), H + min(0, di))
    tj = slice(max(0, dj), W + min(0, dj))
    y[..., si, sj] = x[..., ti, tj]
    return y


def selective_nd_scan_bwd(u, delta, A, B, C, D, delta_bias, dout, delta_softplus=False,
                          A_decay=None, sd=True):
    """Hand adjoint.  Returns the reference's 8-tuple (host.cpp:432):
    du[Bt,Dm,H,W], ddelta[Bt,Dd,H,W], dA[Dm,N], dB, dC [Bt,G,N,H,W], dD[Dm]|None,
    ddelta_bias[Dd]|None, dA_decay[1]|None  (all float64)."""
    u, raw, dl, A, Bc, Cc, a, bu, Dv, adec, dims = _prep(u, delta, A, B, C, D, delta_bias,
                                                        delta_softplus, A_decay)
    Bt, Dm, H, W, Dd, G, N, rd, rg = dims
    dout = np.asarray(dout, np.float64)
    h, s = scan_states(a, bu, sd)
    dyC = dout[:, :, None] * Cc                                          # bwd.cuh:469

    # adjoint recurrences, bottom-right to top-left (bwd.cuh:463-469,486-488 and :710,722-724)
    g = np.zeros_like(h)
    gs = np.zeros_like(h)
    zero = np.zeros(h.shape[:-2])
    for i in range(H - 1, -1, -1):
        for j in range(W - 1, -1, -1):
            acc = dyC[..., i, j].copy()
            if j + 1 < W:
                acc += a[..., i, j + 1] * g[..., i, j + 1]
            if i + 1 < H:
                acc += a[..., i + 1, j] * g[..., i + 1, j]
            if i + 1 < H and j + 1 < W:
                acc -= WEIGHT_LT_H * a[..., i + 1, j + 1] * (a[..., i, j + 1] + a[..., i + 1, j]) \
                    * g[..., i + 1, j + 1]
            g[..., i, j] = acc
            if sd:
                r = gs[..., i, j + 1] * a[..., i, j + 1] if j + 1 < W else zero
                gs[..., i, j] = -dyC[..., i, j] + r

    h_l, h_u, h_d = _shift(h, 0, -1), _shift(h, -1, 0), _shift(h, -1, -1)
    a_l, a_u = _shift(a, 0, -1), _shift(a, -1, 0)
    Y = h_l + h_u - WEIGHT_LT_H * (a_u + a_l) * h_d                      # = (h - bu)/a, bwd.cuh:515
    G_ = a * g
    # total derivative w.r.t. a[i,j]: own multiplier + the two places it enters as a neighbour
    da = g * Y - WEIGHT_LT_H * _shift(G_, 1, 0) * h_l - WEIGHT_LT_H * _shift(G_, 0, 1) * h_u   # bwd.cuh:516-587
    if sd:
        da = da + gs * _shift(s, 0, -1)                                  # bwd.cuh:751-753
        dbu = g + gs + WEIGHT_SELF * dyC                                 # bwd.cuh:750-754
        ystate = h - s + WEIGHT_SELF * bu
    else:
        dbu = g
        ystate = h
    da_a = da * a
    ddl = (da_a * A[None, :, :, None, None]).sum(2) + (dbu * Bc).sum(2) * u          # bwd.cuh:516,752
    du = Dv[None, :, None, None] * dout + (dbu * Bc).sum(2) * dl                      # bwd.cuh:211,514,750
    dA = (da_a * dl[:, :, None]).sum(axis=(0, 3, 4))                                  # bwd.cuh:518,753
    dB = (dbu * (dl * u)[:, :, None]).reshape(Bt, G, rg, N, H, W).sum(2)              # bwd.cuh:589,754
    dC = (dout[:, :, None] * ystate).reshape(Bt, G, rg, N, H, W).sum(2)               # bwd.cuh:590,755
    dD = (dout * u).sum(axis=(0, 2, 3)) if D is not None else None                    # bwd.cuh:212
    dA_decay = np.array([(da_a.sum()) / adec]) if A_decay is not None else None
    if delta_softplus:                                                                # bwd.cuh:785-806
        with np.errstate(over="ignore"):
            ddl = np.where(raw <= SOFTPLUS_THRESHOLD, ddl / (1.0 + np.exp(-raw)), ddl)
    ddelta = ddl.reshape(Bt, Dd, rd, H, W).sum(2)                                     # host.cpp:433-434
    ddelta_bias = ddl.sum(axis=(0, 2, 3)).reshape(Dd, rd).sum(1) if delta_bias is not None else None
    return du, ddelta, dA, dB, dC, dD, ddelta_bias, dA_decay


# --------------------------------------------------------------------------------------------
# Synthetic inputs of the benchmark configurations (value distributions of the headline metric)
# --------------------------------------------------------------------------------------------
def make_inputs(Bt, Dm, H, W, N=16, K=4, seed=0, Dd=None, with_dout=True):
    """u~N(0,1); delta=0.1*N(0,1); delta_bias=log(expm1(dt)), dt log-uniform [1e-3,1e-1];
    A[d,n]=-(n+1); B,C~N(0,1) [Bt,K,N,H,W]; D=1; dout~N(0,1).  float32 numpy arrays."""
    rng = np.random.default_rng(seed)
    Dd = Dm if Dd is None else Dd
    f = np.float32
    u = rng.standard_normal((Bt, Dm, H, W)).astype(f)
    delta = (0.1 * rng.standard_normal((Bt, Dd, H, W))).astype(f)
    dt = np.exp(rng.uniform(np.log(1e-3), np.log(1e-1), size=Dd))
    delta_bias = np.log(np.expm1(dt)).astype(f)
    A = -np.tile(np.arange(1, N + 1, dtype=f)[None], (Dm, 1))
    B = rng.standard_normal((Bt, K, N, H, W)).astype(f)
    C = rng.standard_normal((Bt, K, N, H, W)).astype(f)
    D = np.ones(Dm, f)
    d = dict(u=u, delta=delta, A=A, B=B, C=C, D=D, delta_bias=delta_bias)
    if with_dout:
        d["dout"] = rng.standard_normal((Bt, Dm, H, W)).astype(f)
    return d
