"""Four-corner scanning around the 2D selective scan (the "four-corner multi-directional scanning
strategy that fuses features with trainable weights" of the reference's README.md:45).

The reference kernel scans every group from the top-left corner and leaves the per-group order as a
TODO (selective_scan_fwd_kernel_oflex.cuh:140), so its callers have to materialise the other three
corners: flip copies of the inputs, scan, flip the outputs back.  Two ways to get the same result:

    four_corner_scan(...)            directions=1 inside the HIP kernels: no copies, tensors stay in
                                     their natural orientation (group g starts at corner g % 4)
    four_corner_scan_by_flips(...)   the flip / scan / un-flip construction on top of the
                                     reference-behaviour op; kept as the equivalence check

Channels are laid out direction-major: channel k*C + c is feature c scanned from corner k, group k
of B and C belongs to corner k (G = 4, or a multiple of 4 with group g -> corner g % 4).
"""
import torch

from .interface import selective_nd_scan, selective_nd_scan_merged

# corner k = (rows reversed, columns reversed): 0 top-left, 1 top-right, 2 bottom-left, 3 bottom-right
CORNER_FLIPS = ((False, False), (False, True), (True, False), (True, True))


def _flip(t, k):
    fv, fh = CORNER_FLIPS[k % 4]
    dims = [d for d, on in ((-2, fv), (-1, fh)) if on]
    return torch.flip(t, dims) if dims else t


def flip_groups(t, n_groups):
    """Flip group g of a [B, G*r, H, W] or [B, G, N, H, W] tensor to the orientation of corner g % 4."""
    if t.dim() == 5:
        return torch.stack([_flip(t[:, g], g) for g in range(n_groups)], 1)
    Bt, Dm, H, W = t.shape
    v = t.reshape(Bt, n_groups, Dm // n_groups, H, W)
    return torch.stack([_flip(v[:, g], g) for g in range(n_groups)], 1).reshape(Bt, Dm, H, W)


def cross_scan(x):
    """[B, C, H, W] -> [B, 4*C, H, W]: the feature map once per corner, direction-major, natural
    orientation (what the directions=1 kernels consume)."""
    return x.repeat(1, 4, 1, 1)


def cross_merge(y, weights=None):
    """[B, 4*C, H, W] -> [B, C, H, W]: sum of the four direction outputs, or their fusion with
    trainable weights [4] or [4, C] (README.md:45)."""
    Bt, D4, H, W = y.shape
    v = y.reshape(Bt, 4, D4 // 4, H, W)
    if weights is None:
        return v.sum(1)
    w = weights.reshape(1, 4, -1, 1, 1).to(v.dtype)
    return (v * w).sum(1)


def four_corner_scan(u, delta, A, B, C, D=None, delta_bias=None, delta_softplus=False, out_float=True,
                     A_decay=None):
    """u, delta [B, G*r, H, W], B, C [B, G, N, H, W] in natural orientation; group g is scanned from
    corner g % 4 by the kernels.  u may also be [B, r, H, W]: one feature map shared by the G groups.
    Returns out [B, G*r, H, W] in natural orientation."""
    return selective_nd_scan(u, delta, A, B, C, D, delta_bias, delta_softplus, out_float, A_decay, directions=1)


def four_corner_scan_by_flips(u, delta, A, B, C, D=None, delta_bias=None, delta_softplus=False, out_float=True,
                              A_decay=None):
    """Same result through flipped copies and the top-left-only op (how the reference op is used)."""
    G = B.shape[1]
    if u.shape[1] != A.shape[0]:
        u = u.repeat(1, G, 1, 1)
    out = selective_nd_scan(flip_groups(u, G), flip_groups(delta, G) if delta.shape[1] % G == 0 else delta, A,
                            flip_groups(B, G), flip_groups(C, G), D, delta_bias, delta_softplus, out_float, A_decay)
    return flip_groups(out, G)


def cross_scan_2d(x, delta, A, B, C, D=None, delta_bias=None, delta_softplus=True, merge_weights=None,
                  A_decay=None):
    """The block's scan stage: x [B, C, H, W] is scanned from the four corners (delta [B, 4*C, H, W],
    A [4*C, N], B, C [B, 4, N, H, W], D, delta_bias [4*C] are per direction) and the four results are
    fused into [B, C, H, W] (fp32).  One kernel call each way: x is passed as it is (the kernels let every
    direction group read the same C channels, so not even cross_scan's copies are made), and the four
    results of a feature are added, with their weights, straight into the merged output (no [B, 4*C, H, W]
    tensor is written or read back; the backward reads the merged gradient the same way).
    merge_weights: None, [4] or [4, C]."""
    return selective_nd_scan_merged(x, delta, A, B, C, D, delta_bias, delta_softplus, A_decay, 1, merge_weights)


def cross_scan_2d_unfused(x, delta, A, B, C, D=None, delta_bias=None, delta_softplus=True, merge_weights=None,
                          A_decay=None):
    """cross_scan_2d as two steps (the scan writes [B, 4*C, H, W], cross_merge reduces it): the check of the
    fused path."""
    y = four_corner_scan(x, delta, A, B, C, D, delta_bias, delta_softplus, True, A_decay)
    return cross_merge(y, merge_weights)
