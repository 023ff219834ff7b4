"""A selective state-space mixer in its scalar-decay form (one decay a head and token).

  W_in h = [z: inner | x: inner | B: groups*N | C: groups*N | dt: heads],  inner = heads * head_dim;
  x, B, C pass a causal convolution per channel (taps inputs, the last the token's own; zeros before a sequence's
  start) with a bias, then silu;
  dt <- softplus(dt + dt_bias);  per head h (group h // (heads/groups)):
  S_t = exp(-exp(A_log_h) dt) S_(t-1) + dt B_t x_t^T,   y_t = S_t^T C_t + D_h x_t        S is N x head_dim, from zero;
  y * silu(z), an RMS norm in `norm_groups` equal parts times a weight, the output projection.

Two states per request: the recurrence's [heads, head_dim, N] and the convolution's last taps - 1 inputs
[taps - 1, channels], both float32 rows of the cache manager's pools.  Step sizes, decays, the state, the gate and
the norm are float32 whatever the activations' dtype.
"""
from __future__ import annotations

from typing import Dict, Sequence

import torch

from .. import kernels
from ..cache.needs import FixedState
from .base import BuildContext, Mixer, Param
from .linear import Linear
from .registry import register_mixer


@register_mixer("selective_state_space")
class SelectiveStateSpace(Mixer):
    records_mixed_steps = True

    def __init__(self, hidden_size: int, heads: int, head_dim: int, state_size: int, groups: int, conv_taps: int,
                 norm_groups: int, eps: float, ctx: BuildContext,
                 names: Sequence[str] = ("in", "conv", "conv.b", "dt_bias", "A_log", "D", "norm", "o"), suffix: str = ""):
        self.H, self.dv, self.N, self.G = int(heads), int(head_dim), int(state_size), int(groups)
        self.taps, self.norm_groups, self.eps = int(conv_taps), int(norm_groups), float(eps)
        self.inner = self.H * self.dv
        self.C = self.inner + 2 * self.G * self.N          # channels of the convolution: x | B | C
        if self.G <= 0 or self.H % self.G:
            raise ValueError(f"{self.H} heads do not divide into {self.G} groups")
        if self.norm_groups <= 0 or self.inner % self.norm_groups:
            raise ValueError(f"{self.inner} channels do not divide into {self.norm_groups} norm groups")
        if not 1 <= self.taps <= kernels.CONV_MAX_TAPS:
            raise ValueError(f"{self.taps} taps: the convolution kernel takes 1 to {kernels.CONV_MAX_TAPS}")
        if self.N > kernels.SCAN_MAX_KEY_DIM:
            raise ValueError(f"state size {self.N} is above the recurrence kernel's {kernels.SCAN_MAX_KEY_DIM}")
        self.dtype = ctx.dtype
        self.names = tuple(names)
        self.in_proj = Linear(hidden_size, 2 * self.inner + 2 * self.G * self.N + self.H, names[0], False, ctx, suffix=suffix)
        self.o_proj = Linear(self.inner, hidden_size, names[7], False, ctx, suffix=suffix)
        dev = ctx.device
        self.conv_w = torch.empty((self.C, self.taps), dtype=ctx.dtype, device=dev)
        self.conv_b = torch.empty((self.C,), dtype=ctx.dtype, device=dev)
        self.dt_bias = torch.empty((self.H,), dtype=torch.float32, device=dev)
        self.a_log = torch.empty((self.H,), dtype=torch.float32, device=dev)
        self.skip = torch.empty((self.H,), dtype=torch.float32, device=dev)
        self.norm_w = torch.empty((self.inner,), dtype=ctx.dtype, device=dev)

    def named_parameters(self) -> Dict[str, Param]:
        n = self.names
        out = dict(self.in_proj.named_parameters())
        out.update(self.o_proj.named_parameters())
        out.update({n[1]: Param(self.conv_w), n[2]: Param(self.conv_b), n[3]: Param(self.dt_bias), n[4]: Param(self.a_log),
                    n[5]: Param(self.skip), n[6]: Param(self.norm_w, neutral=1.0)})
        return out

    def cache_need(self):
        return (FixedState((self.taps - 1, self.C), torch.float32), FixedState((self.H, self.dv, self.N), torch.float32))

    def forward(self, x, batch, view):
        conv_view, ssm_view = view
        inner, GN = self.inner, self.G * self.N
        segments = ssm_view.state_in.numel()
        u = self.in_proj.forward(x)                              # [T, z | x | B | C | dt]
        c = kernels.causal_conv(u[:, inner:inner + self.C], self.conv_w, self.conv_b, conv_view.pool, conv_view.state_in,
                                conv_view.state_out, batch.seg_of_token, batch.seg_offsets, segments, "silu")          # float32 [T, x | B | C]
        dt, decay = kernels.ssm_steps(u[:, inner + self.C:], self.dt_bias, self.a_log)
        y = kernels.decay_scan(c[:, inner + GN:], c[:, inner:inner + GN], c[:, :inner], self.H, self.N, self.dv, self.G,
                               ssm_view.pool, ssm_view.state_in, ssm_view.state_out, batch.seg_offsets, segments,
                               decay_t=decay, kscale_t=dt, skip_h=self.skip, max_len=batch.max_q_len)
        y = kernels.group_norm_gate(y, self.norm_w, self.eps, self.norm_groups, gate=u[:, :inner], gate_act="silu",
                                    gate_before=True, out_dtype=self.dtype)
        return self.o_proj.forward(y)
