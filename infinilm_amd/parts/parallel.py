"""Mixers side by side: every branch reads the same input, the result is the weighted sum of their outputs (float32:
it goes to a norm or into the residual sum, not into a product).

`branches` are mixers of any registered kind, `scales` their weights, `names` the sub-names of their tensors.  What
the branches need of the cache is handed on as one tuple (a branch that itself needs a tuple takes as many members),
and the views come back in the same order.
"""
from __future__ import annotations

from typing import Dict, List, Sequence

import torch

from .. import kernels
from ..config.spec import PartSpec
from .base import BuildContext, Mixer, Param, join_name
from .registry import build_mixer, register_mixer


@register_mixer("parallel")
class ParallelMixers(Mixer):
    def __init__(self, branches: Sequence[PartSpec], scales: Sequence[float], names: Sequence[str], ctx: BuildContext):
        if not branches or len(branches) != len(scales) or len(branches) != len(names):
            raise ValueError("branches, scales and names must be equally many, and at least one")
        self.branches = [build_mixer(b, ctx) for b in branches]
        self.scales = [float(s) for s in scales]
        self.names = list(names)
        self.dtype = ctx.dtype
        self._counts: List[int] = []     # members of the cache need each branch takes (-1: a single need, not a tuple)
        for b in self.branches:
            need = b.cache_need()
            self._counts.append(0 if need is None else (len(need) if isinstance(need, (tuple, list)) else -1))

    @property
    def records_mixed_steps(self) -> bool:
        return all(getattr(b, "records_mixed_steps", False) for b in self.branches)

    def named_parameters(self) -> Dict[str, Param]:
        out: Dict[str, Param] = {}
        for sub, b in zip(self.names, self.branches):
            for name, p in b.named_parameters().items():
                out[join_name(sub, name)] = p
        return out

    def cache_need(self):
        flat = []
        for b in self.branches:
            need = b.cache_need()
            if need is not None:
                flat += list(need) if isinstance(need, (tuple, list)) else [need]
        return tuple(flat) if flat else None

    def forward(self, x, batch, view):
        views = list(view) if view is not None else []
        total = None
        at = 0
        for b, n, s in zip(self.branches, self._counts, self.scales):
            if n == 0:
                v = None
            elif n < 0:
                v, at = views[at], at + 1
            else:
                v, at = tuple(views[at:at + n]), at + n
            y = b.forward(x, batch, v)
            if y.dim() != 2:
                raise RuntimeError("a branch of side-by-side mixers must return one [T, hidden] tensor")
            if total is None:
                total, first = y, s
            elif first is not None:
                total, first = kernels.weighted_sum(total, y, first, s, out_dtype=torch.float32), None
            else:
                total = kernels.weighted_sum(total, y, 1.0, s, out_dtype=torch.float32)
        if first is not None:    # a single branch
            total = kernels.weighted_sum(total, total, first, 0.0, out_dtype=torch.float32)
        return total
