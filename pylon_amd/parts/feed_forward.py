"""Gated feed-forward, gate and up fused into one matrix
(/root/reference/src/pylon/model/layers.py:13-27): ``down(silu(gate(h)) * up(h))``."""
from __future__ import annotations

import torch

from ..config.specs import CappedGatedFeedForwardSpec, GatedFeedForwardSpec
from ..kernels import ops, plan
from .base import Part
from .registry import register_part


class GatedFeedForward(Part):
    def __init__(self, spec: GatedFeedForwardSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        if spec.activation != "silu":
            raise ValueError(f"activation {spec.activation!r} is not supported (only 'silu')")
        self.spec = spec
        self.dtype = dtype
        element_size = torch.empty((), dtype=dtype).element_size()
        self.add_param("gate_up", (2 * spec.intermediate_size, spec.hidden_size), dtype, device,
                       row_padding=plan.gated_row_padding(spec.hidden_size, element_size))
        self.add_param("down", (spec.hidden_size, spec.intermediate_size), dtype, device)
        # With biases: those of gate and up enter in the activation kernel, on the product's float32
        # sums; the down projection's is added here, or, if the block says so, left to the residual sum.
        self.defer_output_bias = False
        if spec.bias:
            self.add_param("gate_up_bias", (2 * spec.intermediate_size,), torch.float32, device, role="vector")
            self.add_param("down_bias", (spec.hidden_size,), torch.float32, device, role="vector")

    @property
    def output_bias(self):
        return self.params.get("down_bias")

    def forward(self, h: torch.Tensor, ctx) -> torch.Tensor:
        if not self.spec.bias:
            hidden = ops.linear_glu(h, self.params["gate_up"], out_dtype=self.dtype)
            return ops.linear_for_residual(hidden, self.params["down"], out_dtype=self.dtype)
        sums = ops.linear(h, self.params["gate_up"], out_dtype=torch.float32)
        hidden = ops.gated_act(sums, alpha=1.0, offset=0.0, limit=0.0, out_dtype=self.dtype,
                               bias=self.params["gate_up_bias"])
        out = ops.linear_for_residual(hidden, self.params["down"], out_dtype=self.dtype)
        if self.defer_output_bias:
            return out
        if out.dim() == 3:  # partial sums: the bias joins the first
            ops.add_bias_(out[0], self.params["down_bias"])
            return out
        return ops.add_bias_(out.float() if out.dtype != torch.float32 else out, self.params["down_bias"])


class CappedGatedFeedForward(Part):
    """``down(a(g) * (u + offset))``, ``g = min(gate(h), limit)``, ``u = clamp(up(h), -limit,
    limit)``, ``a(g) = g * sigmoid(alpha * g)``.  As in the plain gated feed-forward, up to 128
    rows the activation works on the float32 sums of the product and its result is rounded
    once; beyond, the library's product is rounded first."""

    def __init__(self, spec: CappedGatedFeedForwardSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        self.spec = spec
        self.dtype = dtype
        element_size = torch.empty((), dtype=dtype).element_size()
        self.add_param("gate_up", (2 * spec.intermediate_size, spec.hidden_size), dtype, device,
                       row_padding=plan.gated_row_padding(spec.hidden_size, element_size))
        self.add_param("down", (spec.hidden_size, spec.intermediate_size), dtype, device)

    def forward(self, h: torch.Tensor, ctx) -> torch.Tensor:
        spec = self.spec
        sums = torch.float32 if h.shape[0] <= ops.SPLIT_ROWS else self.dtype
        gate_up = ops.linear(h, self.params["gate_up"], out_dtype=sums)
        hidden = ops.gated_act(gate_up, alpha=spec.alpha, offset=spec.offset, limit=spec.limit, out_dtype=self.dtype)
        return ops.linear_for_residual(hidden, self.params["down"], out_dtype=self.dtype)


register_part("feed_forward", "gated_mlp", GatedFeedForward, replace=True)
register_part("feed_forward", "capped_gated_mlp", CappedGatedFeedForward, replace=True)
