"""Two mixers side by side: both read the layer's normed input, and the layer adds
``left_scale * left(h) + right_scale * right(h)``.  Either side is any registered mixer, built from
its own spec with its own parameters (under ``left.`` and ``right.``); what the two keep per request
(keys and values of one side, fixed-size states of either) is asked of the cache manager together
and both find it in the run's one cache view.  The weighted sum is formed in float32 from the two
sides' outputs as their products left them (partial sums included) and goes to the residual sum
unrounded."""
from __future__ import annotations

import torch

from ..config.specs import ParallelMixerSpec
from ..kernels import ops
from .base import KVRequirement, Part, requirement_list
from .registry import build_part, register_part


class ParallelMixer(Part):
    def __init__(self, spec: ParallelMixerSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        self.spec = spec
        self.dtype = dtype
        self.left = self.add_child("left", build_part("mixer", spec.left, dtype=dtype, device=device))
        self.right = self.add_child("right", build_part("mixer", spec.right, dtype=dtype, device=device))
        needs = self.cache_requirement() or ()
        if sum(isinstance(need, KVRequirement) for need in needs) > 1:
            raise ValueError("of two mixers side by side at most one keeps keys and values")
        names = [need.name for need in needs if not isinstance(need, KVRequirement)]
        if len(set(names)) != len(names):
            raise ValueError("two mixers side by side keep states of one name: " + ", ".join(sorted(names)))

    def cache_requirement(self):
        needs = requirement_list(self.left.cache_requirement()) + requirement_list(self.right.cache_requirement())
        return needs or None

    def decode_signature(self, rows: int, bound: int) -> tuple:
        out = ("parallel",)
        for side in (self.left, self.right):
            describe = getattr(side, "decode_signature", None)
            out += (("bound", bound),) if describe is None else (describe(rows, bound),)
        return out

    def forward(self, h: torch.Tensor, ctx, cache, stores: bool) -> torch.Tensor:
        left = self.left.forward(h, ctx, cache, stores)
        right = self.right.forward(h, ctx, cache, stores)
        return ops.scaled_sum(left, self.spec.left_scale, right, self.spec.right_scale)


register_part("mixer", "parallel", ParallelMixer, replace=True)
