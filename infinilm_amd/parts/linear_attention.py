"""Linear attention with a fixed decay per head: no softmax, no denominator, a state of fixed size per request.

  q, k [heads, dk], v [heads, dv] from one fused projection of the mixer's input h, with W_g h for the gate;
  an optional activation on q, k and v; an optional rotation of the first `rotary.dims` entries of every q and k head
  (entry i with entry i + dims/2, angle p * base^(-2i/dims) at position p); k times `k_scale`;
  S_t = decay_h S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t            per head, S starts at zero;
  o divided by its root mean square, per head (`norm` = "head") or over all heads together ("all"), times a weight
  if `norm_weight`; times gate_act(W_g h); the output projection.

Two registered kinds differ in these switches alone.  Angles, the rotated q and k, the state, the norm and the gate
are float32 whatever the activations' dtype; the state lives in a row of the cache manager's pool, [heads, dv, dk].
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import torch

from .. import kernels
from ..cache.needs import FixedState
from .base import BuildContext, Mixer, Param
from .linear import FusedLinear, Linear
from .registry import register_mixer


@register_mixer("decay_linear_attention")
class DecayLinearAttention(Mixer):
    records_mixed_steps = True   # every index comes from the batch's device tensors

    def __init__(self, hidden_size: int, heads: int, key_dim: int, value_dim: int, decay: Sequence[float], eps: float,
                 ctx: BuildContext, activation: str = "none", rotary: Optional[dict] = None, k_scale: float = 1.0,
                 norm: str = "head", norm_weight: bool = False, gate_act: str = "silu",
                 names: Sequence[str] = ("q", "k", "v", "g", "o", "norm"), suffix: str = "", whole_output: bool = False):
        self.H, self.dk, self.dv = int(heads), int(key_dim), int(value_dim)
        if len(decay) != self.H:
            raise ValueError(f"{len(decay)} decays for {self.H} heads")
        if norm not in ("head", "all"):
            raise ValueError(f"norm {norm!r}: 'head' or 'all'")
        if self.dk > kernels.SCAN_MAX_KEY_DIM:
            raise ValueError(f"key size {self.dk} is above the recurrence kernel's {kernels.SCAN_MAX_KEY_DIM}")
        self.activation, self.k_scale, self.eps = activation, float(k_scale), float(eps)
        self.norm_groups = self.H if norm == "head" else 1
        self.gate_act = gate_act
        self.whole_output = bool(whole_output)    # never float32 parts still to be summed (see GQAttention)
        self.dtype = ctx.dtype
        kernels.activation_code(activation), kernels.activation_code(gate_act)
        qn, kn, vn, gn, on, self.norm_name = names
        self.proj = FusedLinear(hidden_size, [self.H * self.dk, self.H * self.dk, self.H * self.dv, self.H * self.dv],
                                [qn, kn, vn, gn], False, ctx, suffix=suffix)
        self.o_proj = Linear(self.H * self.dv, hidden_size, on, False, ctx, suffix=suffix)
        self.decay = torch.tensor([float(a) for a in decay], dtype=torch.float32, device=ctx.device)
        self.norm_w = torch.empty((self.H * self.dv,), dtype=ctx.dtype, device=ctx.device) if norm_weight else None
        self.rd, self.freq = 0, None
        if rotary and int(rotary.get("dims", 0)) > 0:
            self.rd = int(rotary["dims"])
            if self.rd % 2 or self.rd > self.dk:
                raise ValueError(f"{self.rd} rotated entries must be even and at most the key size {self.dk}")
            i = torch.arange(self.rd // 2, dtype=torch.float64)
            self.freq = torch.pow(torch.tensor(float(rotary["base"]), dtype=torch.float64), -2.0 * i / self.rd) \
                .to(torch.float32).to(ctx.device)

    def named_parameters(self) -> Dict[str, Param]:
        out = dict(self.proj.named_parameters())
        out.update(self.o_proj.named_parameters())
        if self.norm_w is not None:
            out[self.norm_name] = Param(self.norm_w, neutral=1.0)
        return out

    def cache_need(self):
        return FixedState((self.H, self.dv, self.dk), torch.float32)

    def forward(self, x, batch, view):
        H, dk, dv = self.H, self.dk, self.dv
        rows = self.proj.forward(x)                                    # [T, q | k | v | g]
        f = kernels.linear_attention_inputs(rows, batch.positions, self.freq, H, dk, dv, self.rd, self.activation, self.k_scale)
        o = kernels.decay_scan(f[:, :H * dk], f[:, H * dk:2 * H * dk], f[:, 2 * H * dk:], H, dk, dv, H, view.pool,
                               view.state_in, view.state_out, batch.seg_offsets, view.state_in.numel(), decay_h=self.decay,
                               max_len=batch.max_q_len)
        y = kernels.group_norm_gate(o, self.norm_w, self.eps, self.norm_groups, gate=rows[:, 2 * H * dk + H * dv:],
                                    gate_act=self.gate_act, out_dtype=self.dtype)
        return self.o_proj.forward(y, allow_parts=not self.whole_output)


@register_mixer("retention")
class Retention(DecayLinearAttention):
    """Rotated q and k, k / sqrt(dk), each head's output of unit root mean square (no weight), gate silu."""

    def __init__(self, hidden_size, heads, key_dim, value_dim, decay, eps, rotary, ctx, **names):
        super().__init__(hidden_size, heads, key_dim, value_dim, decay, eps, ctx, activation="none", rotary=rotary,
                         k_scale=float(key_dim) ** -0.5, norm="head", norm_weight=False, gate_act="silu", **names)


@register_mixer("lightning_attention")
class LightningAttention(DecayLinearAttention):
    """silu on q, k and v, no rotation and no scale, one weighted norm over all heads, gate sigmoid."""

    def __init__(self, hidden_size, heads, key_dim, value_dim, decay, eps, ctx, **names):
        super().__init__(hidden_size, heads, key_dim, value_dim, decay, eps, ctx, activation="silu", rotary=None,
                         k_scale=1.0, norm="all", norm_weight=True, gate_act="sigmoid", **names)


@register_mixer("gated_linear_attention")
class GatedLinearAttention(Mixer):
    """Linear attention whose state decays per key channel by a gate computed from the input:

      q = W_q h / sqrt(dk), k = W_k h [heads, dk], v = W_v h [heads, dv]
      alpha = sigmoid(W_a2 (W_a1 h) + b)^(1/tau)  [heads, dk]      a low-rank pair of projections
      S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t      per head, S [dk, dv] starts at zero
      o RMS-normed per head over dv with a weight [dv] shared by the heads, times silu(W_g h), then W_o.

    The 1/sqrt(dk) is applied to k instead of q (the state is linear in k).  Decays, state, norm and gate are float32
    whatever the activations' dtype; the state lives in a row of the cache manager's pool, [heads, dv, dk].  The low rank
    is the number of rows of W_a1."""
    records_mixed_steps = True

    def __init__(self, hidden_size: int, heads: int, key_dim: int, value_dim: int, decay_rank: int, tau: float, eps: float,
                 ctx: BuildContext, names: Sequence[str] = ("q", "k", "v", "g", "a1", "a2", "o", "norm"), suffix: str = "",
                 bias_suffix: str = "bias", whole_output: bool = False):
        self.H, self.dk, self.dv, self.low = int(heads), int(key_dim), int(value_dim), int(decay_rank)
        if self.dk > kernels.SCAN_MAX_KEY_DIM:
            raise ValueError(f"key size {self.dk} is above the recurrence kernel's {kernels.SCAN_MAX_KEY_DIM}")
        if tau <= 0:
            raise ValueError(f"tau {tau} must be positive")
        self.tau, self.eps = float(tau), float(eps)
        self.whole_output = bool(whole_output)
        self.dtype = ctx.dtype
        qn, kn, vn, gn, a1n, a2n, on, self.norm_name = names
        H, dk, dv = self.H, self.dk, self.dv
        self.proj = FusedLinear(hidden_size, [H * dk, H * dk, H * dv, H * dv, self.low], [qn, kn, vn, gn, a1n], False, ctx, suffix=suffix)
        self.a2 = Linear(self.low, H * dk, a2n, True, ctx, suffix=suffix, bias_suffix=bias_suffix)
        self.o_proj = Linear(H * dv, hidden_size, on, False, ctx, suffix=suffix)
        self.norm_w = torch.empty((dv,), dtype=ctx.dtype, device=ctx.device)
        self._norm_all = None     # (version, the weight once for every head)

    def named_parameters(self) -> Dict[str, Param]:
        out = dict(self.proj.named_parameters())
        out.update(self.a2.named_parameters())
        out.update(self.o_proj.named_parameters())
        out[self.norm_name] = Param(self.norm_w, neutral=1.0)
        return out

    def cache_need(self):
        return FixedState((self.H, self.dv, self.dk), torch.float32)

    def _norm_weight(self) -> torch.Tensor:
        held = self._norm_all
        if held is None or held[0] != (self.norm_w._version, self.norm_w.data_ptr()):
            held = self._norm_all = ((self.norm_w._version, self.norm_w.data_ptr()), self.norm_w.repeat(self.H).contiguous())
        return held[1]

    def forward(self, x, batch, view):
        H, dk, dv = self.H, self.dk, self.dv
        rows = self.proj.forward(x)                                    # [T, q | k | v | g | low]
        g0 = 2 * H * dk + H * dv
        # the low-rank pair's second product without its bias (float32 result), the bias inside the decays' kernel
        z = kernels.gemm(rows[:, g0 + H * dv:], self.a2.weight, None, 1.0, torch.float32)          # [T, heads * dk]
        alpha = kernels.sigmoid_root(z, self.tau, bias=self.a2.bias)
        f = kernels.linear_attention_inputs(rows, None, None, H, dk, dv, 0, "none", float(dk) ** -0.5)
        o = kernels.decay_scan(f[:, :H * dk], f[:, H * dk:2 * H * dk], f[:, 2 * H * dk:], H, dk, dv, H, view.pool,
                               view.state_in, view.state_out, batch.seg_offsets, view.state_in.numel(), decay_c=alpha,
                               max_len=batch.max_q_len)
        y = kernels.group_norm_gate(o, self._norm_weight(), self.eps, H, gate=rows[:, g0:g0 + H * dv], gate_act="silu",
                                    out_dtype=self.dtype)
        return self.o_proj.forward(y, allow_parts=not self.whole_output)
