"""A short causal convolution over time, added to its input: ``h + conv(h)`` with
``conv(h)[t] = sum_j w[:, j] * h[t - taps + 1 + j]`` per channel and zeros before a request's
first token.  A request's last ``taps - 1`` inputs are state of fixed size, kept in its state
slot, so a request can arrive in portions of any size."""
from __future__ import annotations

import torch

from ..config.specs import ShortConvSpec, TokenShiftSpec
from ..kernels import ops
from .base import Part, StateRequirement
from .registry import register_part

STATE_NAME = "conv"


class ShortConv(Part):
    def __init__(self, spec: ShortConvSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        if not 1 <= spec.taps <= 8:
            raise ValueError(f"a short convolution has 1 to 8 taps, got {spec.taps}")
        self.spec = spec
        self.dtype = dtype
        self.add_param("weight", (spec.dim, spec.taps), dtype, device)

    def cache_requirement(self):
        if self.spec.taps == 1:
            return None
        return StateRequirement((self.spec.taps - 1, self.spec.dim), torch.float32, name=STATE_NAME)

    def forward(self, h: torch.Tensor, ctx, cache) -> torch.Tensor:
        state = cache.states[STATE_NAME] if self.spec.taps > 1 else None
        return ops.short_conv(h, self.params["weight"], state, ctx.row_start, ctx.row_slots, rows=ctx.rows,
                              max_count=ctx.max_count, out_dtype=self.dtype)


class TokenShift(Part):
    """``h + (h' - h) * w`` with ``h'`` the previous token's ``h`` (zeros before a request's first
    token) and ``w`` one learned number per channel, in float32 and rounded once.  A request's last
    input is state of fixed size in its state slot, so a request can arrive in portions of any size."""

    STATE = "shift"

    def __init__(self, spec: TokenShiftSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        self.spec = spec
        self.dtype = dtype
        self.add_param("weight", (spec.dim,), torch.float32, device, role="vector")

    def cache_requirement(self):
        return StateRequirement((self.spec.dim,), torch.float32, name=self.STATE)

    def forward(self, h: torch.Tensor, ctx, cache) -> torch.Tensor:
        return ops.token_shift(h, self.params["weight"], cache.states[self.STATE], ctx.row_start, ctx.row_slots,
                               rows=ctx.rows, max_count=ctx.max_count, out_dtype=self.dtype)


register_part("conv", "short_conv", ShortConv, replace=True)
register_part("conv", "token_shift", TokenShift, replace=True)
