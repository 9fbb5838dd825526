"""The gated delta rule: linear attention whose state forgets by a learned, input-dependent decay
and is corrected towards every token's value.

``[q; k; v; g; b; a] = W h`` in one product (float32 sums); q, k and v pass a short causal convolution
per channel and ``silu``; per head q and k become unit vectors (q also times ``head_dim ** -0.5``),
``beta = sigmoid(b)``, ``decay = exp(-exp(A_log) * softplus(a + dt_bias))``; per request and head a
float32 state goes from token to token, ``S <- decay S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q``;
every head's ``o`` is divided by its root mean square, multiplied by a weight shared by the heads and
by ``silu(g)``, and projected.  q and k may have fewer heads than v (head ``h`` uses ``h // (n_heads /
n_kv_heads)``).  The state and the convolution's last ``taps - 1`` inputs live in the request's state
slot and start at zero; everything between the projection and the output's rounding is float32
whatever the model's element type."""
from __future__ import annotations

import torch

from ..config.specs import DeltaRuleSpec
from ..kernels import ops
from .base import Part, StateRequirement
from .registry import register_part

STATE = "delta"
CONV_STATE = "delta_conv"


class GatedDeltaRule(Part):
    def __init__(self, spec: DeltaRuleSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        if spec.n_heads < 1 or spec.n_kv_heads < 1 or spec.n_heads % spec.n_kv_heads:
            raise ValueError("The number of value heads must be divisible by the number of q/k heads.")
        if not ops.delta_rule_ok(spec.head_dim, spec.v_head_dim):
            raise ValueError(f"the delta rule does not take heads of {spec.head_dim} x {spec.v_head_dim} elements")
        if not 1 <= spec.conv_taps <= 8:
            raise ValueError(f"a short convolution has 1 to 8 taps, got {spec.conv_taps}")
        self.spec = spec
        self.dtype = dtype
        qk, v = spec.n_kv_heads * spec.head_dim, spec.n_heads * spec.v_head_dim
        self.conv_size = 2 * qk + v                   # channels that pass the convolution: q, k, v
        self.gate_off = self.conv_size                # then the output gate,
        self.beta_off = self.gate_off + v             # a logit of beta per head,
        self.decay_off = self.beta_off + spec.n_heads  # and one of the decay
        self.add_param("proj", (self.decay_off + spec.n_heads, spec.hidden_size), dtype, device)
        self.add_param("conv", (self.conv_size, spec.conv_taps), torch.float32, device, role="vector")
        self.add_param("a_log", (spec.n_heads,), torch.float32, device, role="vector")
        self.add_param("dt_bias", (spec.n_heads,), torch.float32, device, role="vector")
        self.add_param("norm", (spec.v_head_dim,), torch.float32, device, role="vector")
        self.add_param("out", (spec.hidden_size, v), dtype, device)

    def cache_requirement(self):
        spec = self.spec
        # the state transposed: a column of S (one value element) is contiguous
        needs = (StateRequirement((spec.n_heads, spec.v_head_dim, spec.head_dim), torch.float32, name=STATE),)
        if spec.conv_taps > 1:
            needs += (StateRequirement((spec.conv_taps - 1, self.conv_size), torch.float32, name=CONV_STATE),)
        return needs

    def decode_signature(self, rows: int, bound: int) -> tuple:
        return ("delta_rule",)  # nothing of its launches depends on the requests' lengths

    def forward(self, h: torch.Tensor, ctx, cache, stores: bool) -> torch.Tensor:
        spec = self.spec
        if not stores:
            raise ValueError("a delta-rule layer cannot borrow another run's state")
        proj = ops.linear(h, self.params["proj"], out_dtype=torch.float32)
        window = cache.states[CONV_STATE] if spec.conv_taps > 1 else None
        qkv = ops.short_conv(proj[:, : self.conv_size], self.params["conv"], window, ctx.row_start, ctx.row_slots,
                             rows=ctx.rows, max_count=ctx.max_count, out_dtype=torch.float32, mode="silu")
        mixed = ops.delta_rule(
            qkv, proj, cache.states[STATE], self.params["a_log"], self.params["dt_bias"], self.params["norm"],
            ctx.row_start, ctx.row_slots, rows=ctx.rows, heads=spec.n_heads, kv_heads=spec.n_kv_heads,
            dim=spec.head_dim, vdim=spec.v_head_dim, gate_off=self.gate_off, beta_off=self.beta_off,
            decay_off=self.decay_off, eps=spec.norm_eps, unit_eps=spec.unit_eps, q_scale=spec.head_dim ** -0.5,
            out_dtype=self.dtype, max_count=ctx.max_count)
        return ops.linear_for_residual(mixed, self.params["out"], out_dtype=self.dtype)


register_part("mixer", "delta_rule", GatedDeltaRule, replace=True)
