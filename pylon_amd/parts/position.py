"""Position encodings a mixer can be given.

``rope`` follows /root/reference/src/pylon/model/layers.py:43-51 and :73-78: frequencies
``theta ** (-2i/d)`` formed in float32, the angle of a token is ``position * frequency``
(float32), and element ``i`` of a head is rotated together with element ``i + d/2``.
The reference gathers cos/sin from tables of ``max_position_embeddings`` rows; here the
fused q/k kernel forms the angle from the position, which gives the same float32 value.
With ``interleaved`` element ``2i`` is rotated together with its neighbour ``2i + 1`` instead
(the part's ``interleaved`` attribute says so to the mixer, which picks a kernel that does it).
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from ..config.specs import PositionSpec, SinusoidPositionSpec
from ..kernels import ops
from .base import Part
from .registry import register_part


class RotaryPosition(Part):
    def __init__(self, spec: PositionSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        if spec.rotary_dim < 2 or spec.rotary_dim % 2:
            raise ValueError("rotary_dim must be even and at least 2")
        self.spec = spec
        self.interleaved = spec.interleaved
        self.rot_scale = 1.0  # what every cosine and sine is multiplied by
        if spec.scaling is not None:
            inv_freq, self.rot_scale = scaled_frequencies(spec)
        elif spec.interleaved:
            # neighbours (2i, 2i + 1) turn together; frequencies theta ** (-2i/d) formed in double
            # precision and rounded to float32 once
            exponents = torch.arange(0, spec.rotary_dim, 2, dtype=torch.float64) / spec.rotary_dim
            inv_freq = (torch.tensor(spec.theta, dtype=torch.float64) ** -exponents).to(torch.float32)
        else:
            exponents = torch.arange(0, spec.rotary_dim, 2, dtype=torch.float32) / spec.rotary_dim
            inv_freq = 1.0 / (torch.tensor(spec.theta, dtype=torch.float32) ** exponents)
        self.inv_freq = inv_freq.to(device)

    def rotary(self) -> Optional[Tuple[torch.Tensor, int]]:
        return self.inv_freq, self.spec.rotary_dim


def scaled_frequencies(spec: PositionSpec):
    """``(float32 frequencies of the rotary_dim / 2 pairs, the factor on cosine and sine)`` of a
    rotation whose slow pairs are stretched by ``spec.scaling`` (:class:`RotaryScalingSpec`);
    formed in double precision and rounded once."""
    import math

    sc, dims = spec.scaling, spec.rotary_dim
    if not (sc.factor >= 1.0 and sc.original > 0 and sc.fast > 0 and sc.slow > 0 and spec.theta > 1.0):
        raise ValueError("a scaled rotation needs factor >= 1 and positive original, fast and slow")

    def where(turns: float) -> float:
        return dims * math.log(sc.original / (2.0 * math.pi * turns)) / (2.0 * math.log(spec.theta))

    lo = max(math.floor(where(sc.fast)), 0)
    hi = min(math.ceil(where(sc.slow)), dims - 1)
    index = torch.arange(dims // 2, dtype=torch.float64)
    plain = torch.tensor(spec.theta, dtype=torch.float64) ** (-2.0 * index / dims)
    ramp = ((index - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    freq = plain / sc.factor * ramp + plain * (1.0 - ramp)
    return freq.to(torch.float32), 0.1 * math.log(sc.factor) + 1.0


class NoPosition(Part):
    def __init__(self, spec: PositionSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        self.spec = spec
        self.interleaved = False
        self.rot_scale = 1.0

    def rotary(self):
        return None


class SinusoidPosition(Part):
    """A part of the family "stream": a fixed position vector added to the embedded tokens, element
    ``2i`` the sine and element ``2i + 1`` the cosine of ``position * base**(-2i/dim)``.  The
    frequencies are formed in double precision and rounded to float32 once; the angle is the float32
    product of position and frequency."""

    def __init__(self, spec: SinusoidPositionSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        if spec.dim < 1 or not spec.base > 0:
            raise ValueError("a sinusoidal position vector needs a positive size and base")
        self.spec = spec
        exponents = torch.arange(0, spec.dim, 2, dtype=torch.float64) / spec.dim
        self.freq = (torch.tensor(spec.base, dtype=torch.float64) ** -exponents).to(torch.float32).to(device)

    def forward(self, resid: torch.Tensor, ctx) -> torch.Tensor:
        return ops.add_sinusoid(resid, ctx.positions, self.freq)


register_part("position", "rope", RotaryPosition, replace=True)
register_part("stream", "sinusoid", SinusoidPosition, replace=True)
register_part("position", "none", NoPosition, replace=True)
