"""Python face of the 2D-CrossScan selective scan on MI355X.

The reference ships only the pybind pair `fwd` / `bwd`
(kernels/selective_nd_scan/src/cusoflex/selective_scan_oflex.cpp:442-445); the Python function and
autograd.Function that backbones call are authored here on top of the same pair, with the argument
order of those bindings (selective_scan_oflex.cpp:179-187).

    out = selective_nd_scan(u, delta, A, B, C, D=None, delta_bias=None,
                            delta_softplus=False, out_float=True, A_decay=None)

    u      [B, D, H, W]        fp32 / fp16 / bf16   (or [B, D/G, H, W]: one map shared by the G groups)
    delta  [B, Dd, H, W]       same dtype, D % Dd == 0
    A      [D, N]              fp32, N <= 16
    B, C   [B, G, N, H, W]     same dtype as u, D % G == 0
    D      [D] fp32, delta_bias [Dd] fp32, A_decay [1] fp32 (all optional)
    out    [B, D, H, W]        fp32 if out_float else u.dtype

With directions=0 every group is scanned from the top-left corner, as the reference kernel does
(selective_scan_fwd_kernel_oflex.cuh:140).  directions=1 starts group g at corner g % 4 inside the
kernels (no flipped copies); cross_scan.py builds the four-corner block on top of it.
"""
import torch

from ._ext import ext


def fwd(u, delta, A, B, C, D=None, delta_bias=None, delta_softplus=False, out_float=True, A_decay=None,
        directions=0, schedule=-1, merge=False, merge_weights=None):
    """Reference binding `fwd` -> [out, x, x_v, x_sd] (selective_scan_oflex.cpp:179-187,282).
    schedule: block mapping of this call (-1 = the module default, see set_schedule).
    merge: the CrossMerge fused into the output stores: out is [B, D/G, H, W] fp32, the sum over the G
    groups of merge_weights[channel] * (result of the channel) (merge_weights [D] fp32, None = ones)."""
    return ext().fwd(u, delta, A, B, C, D, delta_bias, delta_softplus, out_float, A_decay, directions, schedule,
                     merge, merge_weights)


def bwd(u, delta, A, B, C, D, delta_bias, dout, x, x_v, delta_softplus, A_decay, x_sd, directions=0, schedule=-1,
        merge=False, merge_weights=None):
    """Reference binding `bwd` -> [du, ddelta, dA, dB, dC, dD, ddelta_bias, dA_decay]
    (selective_scan_oflex.cpp:286-297,432-438).  With merge, dout is the gradient of the merged output
    [B, D/G, H, W] and a ninth tensor follows: merge_weights * d merge_weights, per channel [D]."""
    return ext().bwd(u, delta, A, B, C, D, delta_bias, dout, x, x_v, delta_softplus, A_decay, x_sd, directions,
                     schedule, merge, merge_weights)


def set_schedule(mode):
    """Default block mapping of calls that name none: 0 = chosen by shape, 1 = one block per (batch,
    group, 16-channel chunk) plane, 2 = one block per 8-row strip, strips pipelined, 3 = bands of strips,
    4 = the row-segment wavefront kernels (1-4 states).
    Results do not depend on it (only the order of the atomic sums in dA, dB, dC, dD, ddelta_bias does), but a
    bwd must run the kernel family of the fwd whose saved state it is given (modes 1-3 are one family, 4 the other,
    0 picks by shape): the autograd functions see to that themselves; a bwd on another family's state returns NaN
    gradients, never plausible numbers."""
    ext().set_schedule(int(mode))


def get_schedule():
    """The default block mapping (see set_schedule)."""
    return int(ext().get_schedule())


def set_debug(on=True):
    """After every pipelined launch, read the workspace's error word (one stream sync per call) and raise
    if a block-to-block wait timed out.  Also switched on by SND_CHECK_PIPELINE=1 in the environment."""
    ext().set_debug(bool(on))


def init(device=0):
    """Per-device set-up (kernel attributes).  Optional; call it once before capturing launches into a
    HIP graph or launching from several threads."""
    ext().init(int(device))


def _last_dim_contiguous(t):
    return t if (t is None or t.stride(-1) == 1 or t.size(-1) == 1) else t.contiguous()


class SelectiveNdScanFn(torch.autograd.Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, u, delta, A, B, C, D=None, delta_bias=None, delta_softplus=False, out_float=True,
                A_decay=None, directions=0):
        u, delta, B, C = map(_last_dim_contiguous, (u, delta, B, C))
        # The block mapping is resolved once, here, and the backward is told the same one: the two kernel families keep
        # different saved-state layouts, so a default changed between a forward and its backward must not reach it.
        ctx.schedule = get_schedule()
        out, x, x_v, x_sd = fwd(u, delta, A, B, C, D, delta_bias, delta_softplus, out_float, A_decay, directions, ctx.schedule)
        ctx.delta_softplus = delta_softplus
        ctx.directions = directions
        ctx.has = (D is not None, delta_bias is not None, A_decay is not None)
        ctx.save_for_backward(u, delta, A, B, C, D, delta_bias, A_decay, x, x_v, x_sd)
        return out

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, dout):
        u, delta, A, B, C, D, delta_bias, A_decay, x, x_v, x_sd = ctx.saved_tensors
        dout = _last_dim_contiguous(dout)
        du, ddelta, dA, dB, dC, dD, ddelta_bias, dA_decay = bwd(
            u, delta, A, B, C, D, delta_bias, dout, x, x_v, ctx.delta_softplus, A_decay, x_sd, ctx.directions, ctx.schedule)
        has_D, has_bias, has_decay = ctx.has
        return (du, ddelta, dA, dB, dC, dD if has_D else None, ddelta_bias if has_bias else None,
                None, None, dA_decay if has_decay else None, None)


def selective_nd_scan(u, delta, A, B, C, D=None, delta_bias=None, delta_softplus=False, out_float=True,
                      A_decay=None, directions=0):
    """Differentiable 2D-CrossScan selective scan (forward and backward run on the HIP kernels).
    directions=1: group g of B/C (and its dim/G channels) is scanned from corner g % 4."""
    return SelectiveNdScanFn.apply(u, delta, A, B, C, D, delta_bias, delta_softplus, out_float, A_decay, directions)


# Magnitude below which a merge weight enters the backward as +-1e-20 instead of itself.  The kernels return
# weight * d(weight) (every gradient of the op is linear in the weighted dout, so the weight is applied once,
# where dout is staged); dividing by a weight of exactly 0 would lose d(weight), which is <dout, result> and does
# not vanish with the weight.  With the floor, the other gradients of such a channel come out scaled by 1e-20
# instead of 0: far below one ulp of anything they are added to.
_MERGE_WEIGHT_FLOOR = 1e-20


class SelectiveNdScanMergedFn(torch.autograd.Function):
    """The scan with the CrossMerge fused into its output stores: out [B, D/G, H, W] fp32 is the sum over the
    G groups of merge_weights[g, i] * (result of channel g*(D/G) + i)."""

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, u, delta, A, B, C, D, delta_bias, delta_softplus, A_decay, directions, merge_weights):
        u, delta, B, C = map(_last_dim_contiguous, (u, delta, B, C))
        w = None
        if merge_weights is not None:
            G = B.shape[1]
            w = merge_weights.detach().to(torch.float32).reshape(G, -1).expand(G, A.shape[0] // G).contiguous().view(-1)
        ctx.schedule = get_schedule()               # (resolved once for the pair: see SelectiveNdScanFn.forward)
        out, x, x_v, x_sd = fwd(u, delta, A, B, C, D, delta_bias, delta_softplus, True, A_decay, directions, ctx.schedule, True, w)
        ctx.delta_softplus = delta_softplus
        ctx.directions = directions
        ctx.has = (D is not None, delta_bias is not None, A_decay is not None)
        ctx.w_shape = None if merge_weights is None else tuple(merge_weights.shape)
        ctx.w_dtype = None if merge_weights is None else merge_weights.dtype
        ctx.save_for_backward(u, delta, A, B, C, D, delta_bias, A_decay, x, x_v, x_sd, w)
        return out

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, dout):
        u, delta, A, B, C, D, delta_bias, A_decay, x, x_v, x_sd, w = ctx.saved_tensors
        dout = _last_dim_contiguous(dout)
        wb = None
        if w is not None:
            floor = torch.full_like(w, _MERGE_WEIGHT_FLOOR)
            wb = torch.where(w.abs() < _MERGE_WEIGHT_FLOOR, floor, w)
        du, ddelta, dA, dB, dC, dD, ddelta_bias, dA_decay, wdw = bwd(
            u, delta, A, B, C, D, delta_bias, dout, x, x_v, ctx.delta_softplus, A_decay, x_sd, ctx.directions, ctx.schedule,
            True, wb)
        dw = None
        if w is not None and ctx.needs_input_grad[10]:
            G = B.shape[1]
            dw = (wdw / wb).view(G, -1)
            if ctx.w_shape != tuple(dw.shape):       # weights were given per group ([G] or [G, 1]): sum the features
                dw = dw.sum(1).view(ctx.w_shape)
            dw = dw.to(ctx.w_dtype)
        has_D, has_bias, has_decay = ctx.has
        return (du, ddelta, dA, dB, dC, dD if has_D else None, ddelta_bias if has_bias else None,
                None, dA_decay if has_decay else None, None, dw)


def selective_nd_scan_merged(u, delta, A, B, C, D=None, delta_bias=None, delta_softplus=False, A_decay=None,
                             directions=1, merge_weights=None):
    """selective_nd_scan followed by the merge of the G group results of every feature, in one kernel call:
    returns [B, D/G, H, W] fp32 = sum_g merge_weights[g, i] * out[:, g*(D/G) + i].  merge_weights: None (plain
    sum), [G], [G, 1] or [G, D/G]; differentiable.  The sum is accumulated with float atomics, so its last bits
    depend on the order the groups arrive in."""
    if merge_weights is not None:
        G = B.shape[1]
        if merge_weights.dim() == 1:
            if merge_weights.numel() != G:
                raise ValueError("merge_weights must have shape [G], [G, 1] or [G, D/G]")
        elif tuple(merge_weights.shape) not in ((G, 1), (G, A.shape[0] // G)):
            raise ValueError("merge_weights must have shape [G], [G, 1] or [G, D/G]")
    return SelectiveNdScanMergedFn.apply(u, delta, A, B, C, D, delta_bias, delta_softplus, A_decay, directions,
                                         merge_weights)
