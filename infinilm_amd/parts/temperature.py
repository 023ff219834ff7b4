"""Positions without rotation: queries and keys of unit root mean square, and a query temperature that grows with
the logarithm of the position.

  q <- q / sqrt(mean(q^2) + eps),  k <- k / sqrt(mean(k^2) + eps)       per head, no weight (`normed`)
  q <- q * (1 + coef * ln(floor((p + 1) / every) + 1))                   at position p (`every` > 0)

A position encoding in the mixers' sense: it is what the attention mixer hands its fused projection to before the
scores are formed, and it writes k and v into the cache in the same pass.  With `normed` off and `every` 0 it only
writes the cache.  `head_dim` is the number of entries of a head that count; a mixer may run heads filled up with
zeros beyond them.
"""
from __future__ import annotations

from .. import kernels
from .base import BuildContext, PositionEncoding
from .registry import register_position_encoding


@register_position_encoding("unit_norm_temperature")
class UnitNormTemperature(PositionEncoding):
    head_dim = 0    # any size the mixer runs: the entries beyond `dim` are zeros

    def __init__(self, dim: int, normed: bool, eps: float, coef: float, every: int, ctx: BuildContext):
        self.dim, self.normed, self.eps = int(dim), bool(normed), float(eps)
        self.coef, self.every = float(coef), int(every)
        if self.every < 0:
            raise ValueError(f"a temperature every {every} positions")

    def encode_and_store(self, qkv, batch, view, nh: int, nkv: int, d: int) -> None:
        kernels.unit_qk_kvwrite(qkv, batch.positions, view.k, view.v, view.slots, nh, nkv, d, self.dim, self.normed, self.eps,
                                self.coef, self.every)
