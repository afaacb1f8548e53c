"""Pins for the CPU oracle (oracle/snd_oracle.py).

The reference ships no tests, fixtures or golden vectors for selective_nd_scan, so the oracle is
pinned by what the mathematics fixes: special cases that reduce to textbook routines, closed forms,
symmetries, an independent linear-system solve, hand-expanded tiny grids, and for the adjoint
torch.autograd through an independent torch restatement plus central finite differences.
Each check is chosen so that a dropped term, a wrong sign/index or a transposed operand fails it.
"""
import numpy as np
import pytest
import torch

from oracle import snd_oracle as O
from oracle.snd_torch_ref import selective_nd_scan_torch


def rnd(shape, rng, scale=1.0):
    return rng.standard_normal(shape) * scale


def small_inputs(Bt=2, Dm=4, H=5, W=6, N=3, G=2, Dd=None, seed=0, positive_delta=True):
    rng = np.random.default_rng(seed)
    Dd = Dm if Dd is None else Dd
    u = rnd((Bt, Dm, H, W), rng)
    delta = np.abs(rnd((Bt, Dd, H, W), rng, 0.5)) + 0.05 if positive_delta else rnd((Bt, Dd, H, W), rng, 0.5)
    A = -np.abs(rnd((Dm, N), rng)) - 0.1
    B = rnd((Bt, G, N, H, W), rng)
    C = rnd((Bt, G, N, H, W), rng)
    D = rnd((Dm,), rng)
    bias = rnd((Dd,), rng, 0.3)
    return u, delta, A, B, C, D, bias


# ------------------------------------------------------------------ hand-expanded 2x2 grid
def test_two_by_two_hand_expansion():
    """fwd.cuh:263-272 written out for a 2x2 plane, one channel, one state."""
    rng = np.random.default_rng(1)
    u = rnd((1, 1, 2, 2), rng)
    dl = np.abs(rnd((1, 1, 2, 2), rng)) + 0.1
    A = np.array([[-0.7]])
    B = rnd((1, 1, 1, 2, 2), rng)
    C = rnd((1, 1, 1, 2, 2), rng)
    D = np.array([0.3])
    a = np.exp(dl[0, 0] * A[0, 0])
    bu = B[0, 0, 0] * dl[0, 0] * u[0, 0]
    h00 = bu[0, 0]
    h01 = a[0, 1] * h00 + bu[0, 1]
    h10 = a[1, 0] * h00 + bu[1, 0]
    h11 = a[1, 1] * (h10 + h01 - 0.5 * (a[0, 1] + a[1, 0]) * h00) + bu[1, 1]
    s00, s10 = bu[0, 0], bu[1, 0]
    s01 = a[0, 1] * s00 + bu[0, 1]
    s11 = a[1, 1] * s10 + bu[1, 1]
    h = np.array([[h00, h01], [h10, h11]])
    s = np.array([[s00, s01], [s10, s11]])
    exp_sd = D[0] * u[0, 0] + C[0, 0, 0] * (h - s + 0.25 * bu)
    exp_nosd = D[0] * u[0, 0] + C[0, 0, 0] * h
    np.testing.assert_allclose(O.selective_nd_scan_fwd(u, dl, A, B, C, D)[0, 0], exp_sd, rtol=1e-13)
    np.testing.assert_allclose(O.selective_nd_scan_fwd(u, dl, A, B, C, D, sd=False)[0, 0], exp_nosd, rtol=1e-13)


# ------------------------------------------------------------------ 1D reductions
def _scan1d_closed_form(dl, A, bu):
    """h_j = sum_{k<=j} exp(A * (S_j - S_k)) bu_k with S = cumsum(dl): the textbook selective scan."""
    S = np.cumsum(dl, axis=-1)
    L = dl.shape[-1]
    h = np.zeros_like(bu)
    for j in range(L):
        for k in range(j + 1):
            h[..., j] += np.exp(A * (S[..., j] - S[..., k])) * bu[..., k]
    return h


def test_single_row_reduces_to_1d_scan():
    u, delta, A, B, C, D, bias = small_inputs(Bt=1, Dm=2, H=1, W=9, N=2, G=1)
    out_nosd, h, s = O.selective_nd_scan_fwd(u, delta, A, B, C, D, sd=False, return_states=True)
    for c in range(2):
        for n in range(2):
            bu = B[0, 0, n, 0] * delta[0, c, 0] * u[0, c, 0]
            np.testing.assert_allclose(h[0, c, n, 0], _scan1d_closed_form(delta[0, c, 0], A[c, n], bu), rtol=1e-12)
    # with the SD branch a single row has h == s, so only the quarter self term survives
    out_sd = O.selective_nd_scan_fwd(u, delta, A, B, C, D, sd=True)
    Bc = np.repeat(B, 2, axis=1)
    Cc = np.repeat(C, 2, axis=1)
    expect = D[None, :, None, None] * u + 0.25 * (Cc * Bc * (delta * u)[:, :, None]).sum(2)
    np.testing.assert_allclose(out_sd, expect, rtol=1e-12, atol=1e-14)


def test_single_column_reduces_to_1d_scan():
    u, delta, A, B, C, D, bias = small_inputs(Bt=1, Dm=2, H=8, W=1, N=2, G=1)
    out, h, s = O.selective_nd_scan_fwd(u, delta, A, B, C, D, sd=True, return_states=True)
    Bc = np.repeat(B, 2, axis=1)
    Cc = np.repeat(C, 2, axis=1)
    bu = Bc * (delta * u)[:, :, None]
    np.testing.assert_allclose(s, bu, rtol=0, atol=0)           # row scans of length 1
    for c in range(2):
        for n in range(2):
            np.testing.assert_allclose(
                h[0, c, n, :, 0], _scan1d_closed_form(delta[0, c, :, 0], A[c, n], bu[0, c, n, :, 0]), rtol=1e-12)
    expect = D[None, :, None, None] * u + (Cc * (h - 0.75 * bu)).sum(2)
    np.testing.assert_allclose(out, expect, rtol=1e-12)


# ------------------------------------------------------------------ closed forms
def test_constant_a_is_separable_geometric_filter():
    rng = np.random.default_rng(3)
    H, W = 6, 7
    alpha = 0.8
    a = np.full((H, W), alpha)
    bu = rnd((H, W), rng)
    h, _ = O.scan_states(a, bu, sd=False)
    expect = np.zeros((H, W))
    for i in range(H):
        for j in range(W):
            for p in range(i + 1):
                for q in range(j + 1):
                    expect[i, j] += alpha ** ((i - p) + (j - q)) * bu[p, q]
    np.testing.assert_allclose(h, expect, rtol=1e-12)


def test_antidiagonal_constant_a_closed_form():
    """a[i,j] = f(i+j): h[i,j] = sum_{p<=i,q<=j} bu[p,q] * prod_{t=p+q+1}^{i+j} f(t)."""
    rng = np.random.default_rng(4)
    H, W = 5, 6
    f = rng.uniform(0.3, 0.95, size=H + W)
    a = np.array([[f[i + j] for j in range(W)] for i in range(H)])
    bu = rnd((H, W), rng)
    h, _ = O.scan_states(a, bu, sd=False)
    expect = np.zeros((H, W))
    for i in range(H):
        for j in range(W):
            for p in range(i + 1):
                for q in range(j + 1):
                    expect[i, j] += bu[p, q] * np.prod(f[p + q + 1:i + j + 1])
    np.testing.assert_allclose(h, expect, rtol=1e-12)


def test_linear_system_solve_matches_recurrence():
    """(I - L) h = bu solved densely: an evaluation order unrelated to the row-major loop."""
    rng = np.random.default_rng(5)
    H, W = 4, 5
    a = rng.uniform(0.2, 0.99, size=(H, W))
    bu = rnd((H, W), rng)
    n = H * W
    L = np.zeros((n, n))
    idx = lambda i, j: i * W + j
    for i in range(H):
        for j in range(W):
            if j > 0:
                L[idx(i, j), idx(i, j - 1)] += a[i, j]
            if i > 0:
                L[idx(i, j), idx(i - 1, j)] += a[i, j]
            if i > 0 and j > 0:
                L[idx(i, j), idx(i - 1, j - 1)] -= a[i, j] * 0.5 * (a[i - 1, j] + a[i, j - 1])
    expect = np.linalg.solve(np.eye(n) - L, bu.reshape(-1)).reshape(H, W)
    h, s = O.scan_states(a, bu, sd=True)
    np.testing.assert_allclose(h, expect, rtol=1e-11)
    # SD branch = independent 1D scans per row
    for i in range(H):
        acc = 0.0
        for j in range(W):
            acc = a[i, j] * acc + bu[i, j]
            assert abs(s[i, j] - acc) < 1e-13


def test_transpose_symmetry_of_main_recurrence():
    rng = np.random.default_rng(6)
    a = rng.uniform(0.2, 0.99, size=(5, 7))
    bu = rnd((5, 7), rng)
    h, _ = O.scan_states(a, bu, sd=False)
    ht, _ = O.scan_states(a.T.copy(), bu.T.copy(), sd=False)
    np.testing.assert_allclose(ht.T, h, rtol=1e-13)


def test_linearity_in_u_and_plane_independence():
    u, delta, A, B, C, D, bias = small_inputs()
    rng = np.random.default_rng(7)
    u2 = rnd(u.shape, rng)
    f = lambda uu: O.selective_nd_scan_fwd(uu, delta, A, B, C, D, bias, True)
    np.testing.assert_allclose(f(2.0 * u - 3.0 * u2), 2.0 * f(u) - 3.0 * f(u2), rtol=1e-11, atol=1e-12)
    # changing channel 0 of u must not change any other channel's output
    u3 = u.copy()
    u3[:, 0] += 1.0
    o1, o3 = f(u), f(u3)
    np.testing.assert_array_equal(o1[:, 1:], o3[:, 1:])
    assert np.abs(o1[:, 0] - o3[:, 0]).max() > 1e-3


def test_softplus_bias_and_precomputed_delta_agree():
    u, delta, A, B, C, D, bias = small_inputs(positive_delta=False)
    raw = delta + bias[None, :, None, None]
    sp = np.log1p(np.exp(raw))
    o1 = O.selective_nd_scan_fwd(u, delta, A, B, C, D, bias, True)
    o2 = O.selective_nd_scan_fwd(u, sp, A, B, C, D, None, False)
    np.testing.assert_allclose(o1, o2, rtol=1e-12)
    # threshold: above 20 softplus is the identity (fwd.cuh:223)
    big = np.full_like(delta, 25.0)
    o3 = O.selective_nd_scan_fwd(u, big, A, B, C, D, None, True)
    o4 = O.selective_nd_scan_fwd(u, big, A, B, C, D, None, False)
    np.testing.assert_array_equal(o3, o4)


def test_group_and_delta_group_mapping():
    """channel c uses B/C group c // (Dm/G) and delta group c // (Dm/Dd)  (fwd.cuh:105-106)."""
    u, delta, A, B, C, D, bias = small_inputs(Bt=1, Dm=4, H=3, W=4, N=2, G=2, Dd=2)
    out = O.selective_nd_scan_fwd(u, delta, A, B, C, D, bias, True)
    for c in range(4):
        g, dg = c // 2, c // 2
        single = O.selective_nd_scan_fwd(u[:, c:c + 1], delta[:, dg:dg + 1], A[c:c + 1], B[:, g:g + 1],
                                         C[:, g:g + 1], D[c:c + 1], bias[dg:dg + 1], True)
        np.testing.assert_allclose(out[:, c], single[:, 0], rtol=1e-13)


def test_a_decay_scales_a():
    u, delta, A, B, C, D, bias = small_inputs(Bt=1, Dm=2, H=3, W=3, N=2, G=1)
    dec = 0.9
    o1, h1, _ = O.selective_nd_scan_fwd(u, delta, A, B, C, D, A_decay=np.array([dec]), return_states=True)
    a = np.exp(delta[:, :, None] * A[None, :, :, None, None]) * dec
    bu = np.repeat(B, 2, axis=1) * (delta * u)[:, :, None]
    h2, _ = O.scan_states(a, bu)
    np.testing.assert_allclose(h1, h2, rtol=1e-13)


# ------------------------------------------------------------------ adjoint
def _torch_grads(u, delta, A, B, C, D, bias, dout, softplus, A_decay, sd):
    t = lambda x: None if x is None else torch.tensor(np.asarray(x), dtype=torch.float64, requires_grad=True)
    tu, td, tA, tB, tC, tD, tb, tdec = map(t, (u, delta, A, B, C, D, bias, A_decay))
    out = selective_nd_scan_torch(tu, td, tA, tB, tC, tD, tb, softplus, tdec, sd)
    out.backward(torch.tensor(dout, dtype=torch.float64))
    g = lambda x: None if x is None else x.grad.numpy()
    return out.detach().numpy(), (g(tu), g(td), g(tA), g(tB), g(tC), g(tD), g(tb), g(tdec))


@pytest.mark.parametrize("sd", [True, False])
@pytest.mark.parametrize("softplus,use_bias,use_D,use_decay,Dd", [
    (True, True, True, False, None),
    (False, False, False, False, None),
    (True, True, True, True, 2),
])
def test_hand_adjoint_equals_autograd(sd, softplus, use_bias, use_D, use_decay, Dd):
    u, delta, A, B, C, D, bias = small_inputs(Bt=2, Dm=4, H=5, W=6, N=3, G=2, Dd=Dd, seed=11,
                                              positive_delta=not softplus)
    rng = np.random.default_rng(12)
    dout = rnd(u.shape, rng)
    D_ = D if use_D else None
    b_ = bias if use_bias else None
    dec = np.array([0.93]) if use_decay else None
    out_t, grads_t = _torch_grads(u, delta, A, B, C, D_, b_, dout, softplus, dec, sd)
    out_o = O.selective_nd_scan_fwd(u, delta, A, B, C, D_, b_, softplus, dec, sd)
    np.testing.assert_allclose(out_o, out_t, rtol=1e-12, atol=1e-13)
    grads_o = O.selective_nd_scan_bwd(u, delta, A, B, C, D_, b_, dout, softplus, dec, sd)
    names = ["du", "ddelta", "dA", "dB", "dC", "dD", "ddelta_bias", "dA_decay"]
    for name, go, gt in zip(names, grads_o, grads_t):
        if gt is None:
            assert go is None, name
            continue
        np.testing.assert_allclose(go, gt, rtol=1e-10, atol=1e-12, err_msg=name)


def test_hand_adjoint_finite_differences():
    u, delta, A, B, C, D, bias = small_inputs(Bt=1, Dm=2, H=3, W=4, N=2, G=1, seed=21, positive_delta=False)
    rng = np.random.default_rng(22)
    dout = rnd(u.shape, rng)
    loss = lambda **kw: float((O.selective_nd_scan_fwd(**{**dict(u=u, delta=delta, A=A, B=B, C=C, D=D,
                                                              delta_bias=bias, delta_softplus=True), **kw}) * dout).sum())
    grads = O.selective_nd_scan_bwd(u, delta, A, B, C, D, bias, dout, True)
    eps = 1e-6
    for name, arr, grad in (("u", u, grads[0]), ("delta", delta, grads[1]), ("A", A, grads[2]),
                            ("B", B, grads[3]), ("C", C, grads[4]), ("D", D, grads[5]),
                            ("delta_bias", bias, grads[6])):
        flat = arr.reshape(-1)
        for k in rng.choice(flat.size, size=min(6, flat.size), replace=False):
            p = arr.copy().reshape(-1)
            m = arr.copy().reshape(-1)
            p[k] += eps
            m[k] -= eps
            fd = (loss(**{name: p.reshape(arr.shape)}) - loss(**{name: m.reshape(arr.shape)})) / (2 * eps)
            assert abs(fd - grad.reshape(-1)[k]) <= 1e-6 * max(1.0, abs(fd)), (name, k, fd, grad.reshape(-1)[k])


def test_benchmark_input_generator_shapes():
    d = O.make_inputs(1, 64, 14, 14, N=16, K=4, seed=0)
    assert d["u"].shape == (1, 64, 14, 14) and d["B"].shape == (1, 4, 16, 14, 14)
    assert np.all(d["A"][:, 3] == -4.0) and d["delta_bias"].shape == (64,)
    dt = np.log1p(np.exp(d["delta_bias"].astype(np.float64)))
    assert dt.min() >= 1e-3 * 0.999 and dt.max() <= 1e-1 * 1.001
