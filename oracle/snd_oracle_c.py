"""ctypes front end of the C oracle (oracle/snd_oracle.c).  TEST INFRASTRUCTURE ONLY.

fwd / bwd take and return dense float32 numpy arrays with the reference's layouts
(selective_scan_oflex.cpp:206-229); `real` picks the arithmetic of the state ("f32" = what the
reference computes in, "f64" = checker).
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
_libs = {}
fp = C.POINTER(C.c_float)


def build():
    subprocess.run(["make", "-C", HERE], check=True, stdout=subprocess.DEVNULL)


def lib(real="f32"):
    if real not in _libs:
        path = os.path.join(HERE, "libsnd_oracle_%s.so" % real)
        if not os.path.exists(path):
            build()
        _libs[real] = C.CDLL(path)
    return _libs[real]


def _p(a):
    return None if a is None else a.ctypes.data_as(fp)


def _c(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def fwd(u, delta, A, B, Cc, D=None, delta_bias=None, delta_softplus=False, A_decay=None, real="f32", nthreads=0):
    u, delta, A, B, Cc, D, delta_bias, A_decay = map(_c, (u, delta, A, B, Cc, D, delta_bias, A_decay))
    Bt, Dm, H, W = u.shape
    out = np.empty_like(u)
    lib(real).snd_oracle_fwd(Bt, Dm, H, W, A.shape[1], B.shape[1], delta.shape[1], _p(u), _p(delta), _p(A), _p(B),
                             _p(Cc), _p(D), _p(delta_bias), int(bool(delta_softplus)), _p(A_decay), _p(out),
                             int(nthreads))
    return out


def bwd(u, delta, A, B, Cc, D, delta_bias, dout, delta_softplus=False, A_decay=None, real="f32", nthreads=0):
    """Returns the reference's 8-tuple (selective_scan_oflex.cpp:432-438), float32."""
    u, delta, A, B, Cc, D, delta_bias, A_decay, dout = map(_c, (u, delta, A, B, Cc, D, delta_bias, A_decay, dout))
    Bt, Dm, H, W = u.shape
    N, G, Dd = A.shape[1], B.shape[1], delta.shape[1]
    du, ddelta = np.empty_like(u), np.empty_like(u)
    dA, dB, dC = np.empty_like(A), np.empty_like(B), np.empty_like(Cc)
    dD = np.empty(Dm, np.float32) if D is not None else None
    db = np.empty(Dm, np.float32) if delta_bias is not None else None
    ddec = np.empty(1, np.float32) if A_decay is not None else None
    lib(real).snd_oracle_bwd(Bt, Dm, H, W, N, G, Dd, _p(u), _p(delta), _p(A), _p(B), _p(Cc), _p(D), _p(delta_bias),
                             int(bool(delta_softplus)), _p(A_decay), _p(dout), _p(du), _p(ddelta), _p(dA), _p(dB),
                             _p(dC), _p(dD), _p(db), _p(ddec), int(nthreads))
    if Dd != Dm:                                            # selective_scan_oflex.cpp:433-438
        ddelta = ddelta.reshape(Bt, Dd, Dm // Dd, H, W).sum(2)
        if db is not None:
            db = db.reshape(Dd, Dm // Dd).sum(1)
    return du, ddelta, dA, dB, dC, dD, db, ddec
