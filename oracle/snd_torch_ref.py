"""Differentiable PyTorch restatement of the 2D-CrossScan forward recurrence (CPU, any float dtype).

TEST INFRASTRUCTURE ONLY (same rule as snd_oracle.py: never imported by the shipped package).

Written independently of snd_oracle.py's array code so that torch.autograd through it pins the
hand adjoint there: rows are chained with torch ops, no in-place writes, so autograd sees the
exact dependency graph of
    kernels/selective_nd_scan/include/cusoflex/selective_scan_fwd_kernel_oflex.cuh:189-346.
"""
import torch


def selective_nd_scan_torch(u, delta, A, B, C, D=None, delta_bias=None, delta_softplus=False,
                            A_decay=None, sd=True):
    Bt, Dm, H, W = u.shape
    Dd, G, N = delta.shape[1], B.shape[1], A.shape[1]
    dl = delta.repeat_interleave(Dm // Dd, dim=1)
    if delta_bias is not None:
        dl = dl + delta_bias.repeat_interleave(Dm // Dd)[None, :, None, None]
    if delta_softplus:
        dl = torch.where(dl <= 20.0, torch.log1p(torch.exp(torch.clamp(dl, max=50.0))), dl)
    adec = 1.0 if A_decay is None else A_decay.reshape(-1)[0]
    a = torch.exp(dl[:, :, None] * A[None, :, :, None, None]) * adec       # [Bt,Dm,N,H,W]
    Bc = B.repeat_interleave(Dm // G, dim=1)
    Cc = C.repeat_interleave(Dm // G, dim=1)
    bu = Bc * (dl * u)[:, :, None]
    zero = torch.zeros(Bt, Dm, N, dtype=u.dtype)
    # per-cell views taken once (unbind: its backward is one stack per row, where indexing a[..., i, j] cell by
    # cell would scatter every cell's gradient into a zero tensor of the whole plane)
    ac = [r.unbind(-1) for r in a.unbind(-2)]
    buc = [r.unbind(-1) for r in bu.unbind(-2)]
    rows_h, rows_s = [], []
    for i in range(H):
        hrow, srow = [], []
        for j in range(W):
            left = hrow[j - 1] if j > 0 else zero
            up = rows_h[i - 1][j] if i > 0 else zero
            if i > 0 and j > 0:
                corr = 0.5 * (ac[i - 1][j] + ac[i][j - 1]) * rows_h[i - 1][j - 1]
            else:
                corr = zero
            hrow.append(ac[i][j] * (left + up - corr) + buc[i][j])
            if sd:
                sl = srow[j - 1] if j > 0 else zero
                srow.append(ac[i][j] * sl + buc[i][j])
        rows_h.append(hrow)
        rows_s.append(srow)
    h = torch.stack([torch.stack(r, dim=-1) for r in rows_h], dim=-2)
    if sd:
        s = torch.stack([torch.stack(r, dim=-1) for r in rows_s], dim=-2)
        y = h - s + 0.25 * bu
    else:
        y = h
    out = (Cc * y).sum(2)
    if D is not None:
        out = out + D[None, :, None, None] * u
    return out
