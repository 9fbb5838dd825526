"""RMSNorm over the hidden axis (/root/reference/src/pylon/model/layers.py:30-40):
``y = x / sqrt(mean(x^2) + eps) * w`` in float32, rounded once to the activation dtype.
The weight is kept in float32 whatever the model's dtype, as the reference keeps it.  With
``weight_offset`` the stored weight is a distance from that number: ``y = ... * (offset + w)``."""
from __future__ import annotations

from typing import Optional

import torch

from ..config.specs import NormSpec
from ..kernels import ops
from .base import DepthMixed, Normed, Part, Scaled
from .registry import register_part


class RMSNorm(Part):
    def __init__(self, spec: NormSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        self.spec = spec
        self.dtype = dtype
        self.add_param("weight", (spec.dim,), torch.float32, device, role="vector")
        self._shifted = None  # (version of the parameter, weight + offset)

    def weight(self) -> torch.Tensor:
        """What multiplies: the stored weight, plus ``weight_offset`` for a norm whose weights are
        stored as their distance from it (formed in float32, anew when the parameter is written)."""
        stored = self.params["weight"]
        if not self.spec.weight_offset:
            return stored
        key = (stored.data_ptr(), stored._version)
        if self._shifted is None or self._shifted[0] != key:
            self._shifted = (key, stored + self.spec.weight_offset)
        return self._shifted[1]

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.rmsnorm(x, self.weight(), self.spec.eps, out_dtype=self.dtype)

    def add_forward(self, resid: torch.Tensor, delta, *,
                    row_idx: Optional[torch.Tensor] = None) -> torch.Tensor:
        if isinstance(delta, Normed):
            return ops.add_normed_rmsnorm(resid, delta.value, self.weight(), self.spec.eps, self.dtype,
                                          post_gain=delta.gain, post_eps=delta.eps, row_idx=row_idx)
        if isinstance(delta, DepthMixed):
            # the sum, the layer's result among the streams, their mix and its norm in one kernel;
            # where only some rows are normed, the mix of all rows first
            fused = row_idx is None
            out = ops.depth_mix(resid, delta.value, delta.streams, delta.index, delta.coeff, delta_scale=delta.scale,
                                delta_bias=delta.bias, gain=self.weight() if fused else None, eps=self.spec.eps,
                                out_dtype=self.dtype)
            return out if fused else ops.rmsnorm(resid, self.weight(), self.spec.eps, out_dtype=self.dtype,
                                                 row_idx=row_idx)
        if isinstance(delta, Scaled):
            return ops.add_normed_rmsnorm(resid, delta.value, self.weight(), self.spec.eps, self.dtype,
                                          row_idx=row_idx, delta_scale=delta.scale, delta_bias=delta.bias)
        return ops.add_rmsnorm(resid, delta, self.weight(), self.spec.eps, self.dtype,
                               row_idx=row_idx)


class ScalarRMSNorm(Part):
    """``g * x / sqrt(mean(x^2) + eps)`` with one learned number ``g`` for all coordinates, in
    float32.  As the norm after a sublayer it is not applied here: :meth:`pending` wraps the
    sublayer's output with the gain, and the next norm's kernel norms it, adds it to the residual
    stream and norms the sum in one pass."""

    def __init__(self, spec: NormSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        self.spec = spec
        self.dtype = dtype
        self.add_param("weight", (), torch.float32, device, role="vector")

    def pending(self, value: torch.Tensor) -> Normed:
        return Normed(value, self.params["weight"], self.spec.eps)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.add_normed_rmsnorm(x.float() if x.dtype != torch.float32 else x, None, self.params["weight"],
                                      self.spec.eps, self.dtype)

    def add_forward(self, resid: torch.Tensor, delta, *, row_idx: Optional[torch.Tensor] = None) -> torch.Tensor:
        if isinstance(delta, Normed):
            return ops.add_normed_rmsnorm(resid, delta.value, self.params["weight"], self.spec.eps, self.dtype,
                                          post_gain=delta.gain, post_eps=delta.eps, row_idx=row_idx)
        return ops.add_normed_rmsnorm(resid, delta, self.params["weight"], self.spec.eps, self.dtype, row_idx=row_idx)


register_part("norm", "rmsnorm", RMSNorm, replace=True)
register_part("norm", "scalar_rmsnorm", ScalarRMSNorm, replace=True)
