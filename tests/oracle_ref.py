"""Float64 oracle results for a call with options (corner directions, A_decay, softplus off, absent D / bias,
shared delta groups), for tests that compare HIP kernels with the oracle directly.  Test support only."""
import numpy as np

from oracle import snd_oracle_c as OC


def _flip(a, g):
    """One group's planes to / from the orientation of corner g % 4 (bit 1: rows, bit 0: columns)."""
    if g & 2:
        a = a[..., ::-1, :]
    if g & 1:
        a = a[..., ::-1]
    return a


def flip_groups(a, G):
    """[B, G*r, H, W] or [B, G, N, H, W]: group g to / from the orientation of corner g % 4."""
    if a.ndim == 5:
        return np.ascontiguousarray(np.stack([_flip(a[:, g], g) for g in range(G)], 1))
    Bt, Dm, H, W = a.shape
    v = a.reshape(Bt, G, Dm // G, H, W)
    return np.ascontiguousarray(np.stack([_flip(v[:, g], g) for g in range(G)], 1).reshape(Bt, Dm, H, W))


def reference(u, delta, A, B, C, D, delta_bias, dout, softplus=True, decay=None, corners=False):
    """(out, [du, ddelta, dA, dB, dC, dD, ddelta_bias, dA_decay]) of the float64 C oracle.  With corners, group g is
    scanned from corner g % 4: the oracle scans flipped copies from the top-left and the results are flipped back
    (the per-channel sums dA, dD, ddelta_bias, dA_decay do not depend on the orientation).  delta may have fewer
    channels than u (shared delta groups: flipped per delta channel's group, which needs Dd % G == 0 there)."""
    G = B.shape[1]
    dec = None if decay is None else np.asarray([decay], np.float32)
    f = (lambda a: flip_groups(np.ascontiguousarray(a), G)) if corners else (lambda a: np.ascontiguousarray(a))
    args = (f(u), f(delta), A, f(B), f(C), D, delta_bias)
    out = f(OC.fwd(*args, softplus, dec, real="f64"))
    g = OC.bwd(*args, f(dout), softplus, dec, real="f64")
    return out, [f(g[0]), f(g[1]), g[2], f(g[3]), f(g[4]), g[5], g[6], g[7]]
