"""The C restatement of the oracle (the timed CPU baseline and the checker for large shapes) must
agree with the pinned numpy oracle."""
import numpy as np
import pytest

from oracle import snd_oracle as O
from oracle import snd_oracle_c as OC

NAMES = ["du", "ddelta", "dA", "dB", "dC", "dD", "ddelta_bias", "dA_decay"]


def rel(x, ref):
    s = np.abs(ref).max()
    return float(np.abs(np.asarray(x, np.float64) - ref).max() / (s if s > 1e-12 else 1e-2))


@pytest.mark.parametrize("shape", [(1, 64, 14, 14, 16, 4, None), (2, 12, 9, 11, 5, 3, 4), (1, 4, 1, 19, 16, 1, None),
                                   (1, 4, 13, 1, 16, 2, None)])
@pytest.mark.parametrize("real,tol", [("f64", 2e-6), ("f32", 2e-4)])
def test_c_oracle_matches_numpy_oracle(shape, real, tol):
    Bt, Dm, H, W, N, K, Dd = shape
    d = O.make_inputs(Bt, Dm, H, W, N=N, K=K, seed=3, Dd=Dd)
    dec = np.array([0.95], np.float32)
    args = (d["u"], d["delta"], d["A"], d["B"], d["C"], d["D"], d["delta_bias"])
    ref = O.selective_nd_scan_fwd(*args, True, dec)
    out = OC.fwd(*args, True, dec, real=real, nthreads=4)
    assert rel(out, ref) <= tol
    gref = O.selective_nd_scan_bwd(*args, d["dout"], True, dec)
    g = OC.bwd(*args, d["dout"], True, dec, real=real, nthreads=4)
    for name, a, b in zip(NAMES, g, gref):
        assert a.shape == b.shape, name
        assert rel(a, b) <= tol, (name, rel(a, b))


def test_c_oracle_optional_inputs_absent():
    d = O.make_inputs(1, 4, 6, 7, N=3, K=2, seed=4)
    delta = np.abs(d["delta"]) + 0.02
    ref = O.selective_nd_scan_fwd(d["u"], delta, d["A"], d["B"], d["C"])
    assert rel(OC.fwd(d["u"], delta, d["A"], d["B"], d["C"], real="f64"), ref) <= 2e-6
    g = OC.bwd(d["u"], delta, d["A"], d["B"], d["C"], None, None, d["dout"], real="f64")
    gref = O.selective_nd_scan_bwd(d["u"], delta, d["A"], d["B"], d["C"], None, None, d["dout"])
    assert g[5] is None and g[6] is None and g[7] is None
    for a, b in zip(g[:5], gref[:5]):
        assert rel(a, b) <= 2e-6
