"""A VSS-style block around the four-corner 2D selective scan: the caller that produces the op's
inputs in a 2D-CrossScan backbone.

The reference repository ships only the kernel (README.md:62-69 points at VMamba / SparseFormer for
the models "with minor modifications such as replacing the backbone and kernel"); this module
follows the upstream VMamba SS2D layout of that caller so the op can be dropped into such a block:

    x [B, H, W, C] -> in_proj -> (x, z) -> depthwise 3x3 conv + SiLU
      -> per direction k: x_proj_k -> (dt_k, B_k, C_k), dt_proj_k -> delta_k          (1x1 maps)
      -> four-corner scan (direction k = scan origin corner k, kernel option directions=1)
      -> fuse the four results with trainable weights (README.md:45) -> LayerNorm -> * SiLU(z) -> out_proj

Because the scan origins are handled inside the kernels, every tensor stays in its natural
orientation: the projections are pointwise, so no flipped (or even repeated) copy of the feature
map is ever built - the four direction groups read the same u.
Everything outside the scan is plain PyTorch (GEMMs / elementwise); `scan_fn` can be replaced for
testing.
"""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from .cross_scan import cross_merge, four_corner_scan


class SS2DCrossScan(nn.Module):
    K = 4  # scan origins: the four corners

    def __init__(self, d_model, d_state=16, ssm_ratio=2.0, dt_rank="auto", d_conv=3, conv_bias=True, bias=False,
                 dt_min=1e-3, dt_max=1e-1, dt_init_floor=1e-4, merge="weighted", scan_fn=None):
        super().__init__()
        self.d_model, self.d_state = d_model, d_state
        self.d_inner = int(ssm_ratio * d_model)
        self.dt_rank = math.ceil(d_model / 16) if dt_rank == "auto" else dt_rank
        self.scan_fn = scan_fn or four_corner_scan
        K, Di, N, R = self.K, self.d_inner, d_state, self.dt_rank

        self.in_proj = nn.Linear(d_model, 2 * Di, bias=bias)
        self.conv2d = nn.Conv2d(Di, Di, d_conv, padding=(d_conv - 1) // 2, groups=Di, bias=conv_bias)
        # per-direction projections, stacked on a leading K axis
        self.x_proj_weight = nn.Parameter(torch.empty(K, R + 2 * N, Di))
        nn.init.kaiming_uniform_(self.x_proj_weight.view(-1, Di), a=math.sqrt(5))
        self.dt_projs_weight = nn.Parameter(torch.empty(K, Di, R).uniform_(-R ** -0.5, R ** -0.5))
        dt = torch.exp(torch.rand(K, Di) * (math.log(dt_max) - math.log(dt_min)) + math.log(dt_min)).clamp(min=dt_init_floor)
        self.dt_projs_bias = nn.Parameter(dt + torch.log(-torch.expm1(-dt)))        # softplus^-1(dt)
        self.A_logs = nn.Parameter(torch.log(torch.arange(1, N + 1, dtype=torch.float32)).repeat(K * Di, 1))
        self.Ds = nn.Parameter(torch.ones(K * Di))
        self.merge_weights = nn.Parameter(torch.ones(K, Di)) if merge == "weighted" else None
        self.out_norm = nn.LayerNorm(Di)
        self.out_proj = nn.Linear(Di, d_model, bias=bias)

    def scan_inputs(self, x):
        """x [B, Di, H, W] (after conv + activation) -> (u, delta, A, B, C, D, delta_bias) of the op."""
        Bt, Di, H, W = x.shape
        K, N, R = self.K, self.d_state, self.dt_rank
        x_dbl = torch.einsum("bdhw,kcd->bkchw", x, self.x_proj_weight.to(x.dtype))
        dts, Bs, Cs = torch.split(x_dbl, [R, N, N], dim=2)
        delta = torch.einsum("bkrhw,kdr->bkdhw", dts, self.dt_projs_weight.to(x.dtype)).reshape(Bt, K * Di, H, W)
        A = -torch.exp(self.A_logs.float())
        return (x, delta.contiguous(), A, Bs.contiguous(), Cs.contiguous(), self.Ds.float(),
                self.dt_projs_bias.float().reshape(-1))

    def forward(self, x):
        """x [B, H, W, d_model] -> [B, H, W, d_model]."""
        xz = self.in_proj(x)
        x, z = xz.chunk(2, dim=-1)
        x = F.silu(self.conv2d(x.permute(0, 3, 1, 2).contiguous()))
        u, delta, A, Bs, Cs, Ds, dt_bias = self.scan_inputs(x)
        ys = self.scan_fn(u, delta, A, Bs, Cs, Ds, dt_bias, True, True)              # [B, K*Di, H, W] fp32
        y = cross_merge(ys, self.merge_weights)                                       # [B, Di, H, W]
        y = self.out_norm(y.permute(0, 2, 3, 1)).to(z.dtype)
        return self.out_proj(y * F.silu(z))


class VSSBlock(nn.Module):
    """Pre-norm residual block: x + SS2D(LN(x)), then x + MLP(LN(x)) when mlp_ratio > 0."""

    def __init__(self, d_model, d_state=16, ssm_ratio=2.0, mlp_ratio=4.0, **ss2d_kwargs):
        super().__init__()
        self.norm = nn.LayerNorm(d_model)
        self.op = SS2DCrossScan(d_model, d_state=d_state, ssm_ratio=ssm_ratio, **ss2d_kwargs)
        self.mlp = None
        if mlp_ratio > 0:
            hidden = int(mlp_ratio * d_model)
            self.norm2 = nn.LayerNorm(d_model)
            self.mlp = nn.Sequential(nn.Linear(d_model, hidden), nn.GELU(), nn.Linear(hidden, d_model))

    def forward(self, x):
        x = x + self.op(self.norm(x))
        if self.mlp is not None:
            x = x + self.mlp(self.norm2(x))
        return x
