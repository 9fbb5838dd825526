"""A mixture of gated feed-forward experts with an optional shared expert.

Router logits ``W_r h + b`` are float32 sums of exact products (``ops.linear`` with a float32
result: bfloat16 operands on the matrix cores with float32 accumulation, never rounded; float32
operands on the exact kernel; with a gated shared expert its gate vector is one more row of the
router's matrix);
one kernel picks every token's ``top`` experts and the softmax over their logits; one computes
``silu(gate) * up`` of every (token, chosen expert) from the experts' fused gate/up matrix, and one
applies the chosen experts' down matrices, weights the results and adds the shared expert's output
times its gate (from 33 bfloat16 tokens on, the (token, expert) pairs are sorted by expert on the
device instead and every expert's pairs run as tiles on the matrix cores).  The shared expert itself is an ordinary gated feed-forward on the engine's
product kernels.  The result is float32 and goes to the residual sum unrounded.  A token's
output does not depend on which other tokens share its step: every kernel here works token by
token with a fixed order of additions.

The spec may ask instead for plain experts ``down(relu(up(h))^2)`` (``expert_act="relu2"``: one
matrix ``up`` in place of ``gate_up``), and for the other way of routing (``scoring="softmax_all"``,
:func:`ops.route_scored`): scores from a softmax over all router outputs, a correction for the choice
only, a choice limited to the best groups of neighbouring outputs, weights that are the scores times a
constant, and identity experts (router outputs without matrices, whose output is the input itself:
the expert kernels pass over them and add the input times the sum of their weights).

``scoring="sigmoid"``: the chosen experts' weights are the sigmoids of their own router outputs, not
renormalised.  ``weight_on_input``: a chosen expert runs on the token's input times its weight,
``sum_e expert_e(w_e h)``; the token-by-token kernel scales the input in float32 as it stages it, the
sorted path scales the gate's and the up's float32 sums before the activation (the same number,
because the two products are linear).
"""
from __future__ import annotations

import torch

from ..config.specs import MixtureFeedForwardSpec
from ..kernels import ops, plan
from .base import Part
from .registry import register_part


class MixtureFeedForward(Part):
    def __init__(self, spec: MixtureFeedForwardSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        choices = spec.n_experts + (spec.n_identity if spec.scoring == "softmax_all" else 0)
        if spec.n_experts < 1 or not 1 <= spec.top <= choices:
            raise ValueError(f"a token uses 1 to {choices} of {choices} experts, not {spec.top}")
        if spec.n_experts > 512 or spec.top > 32:
            raise ValueError("the router kernel takes up to 512 experts and up to 32 of them a token")
        if spec.shared_size is None and spec.shared_gate:
            raise ValueError("a gate of the shared expert needs a shared expert")
        if spec.expert_act not in ops.EXPERT_ACTS:
            raise ValueError(f"unknown activation of the experts {spec.expert_act!r} (known: {', '.join(ops.EXPERT_ACTS)})")
        if spec.scoring not in ("top_softmax", "softmax_all", "sigmoid"):
            raise ValueError(f"unknown scoring {spec.scoring!r} (known: top_softmax, softmax_all, sigmoid)")
        if spec.weight_on_input and (spec.expert_act != "silu_gated" or spec.n_identity):
            raise ValueError("weights on the experts' inputs go with gated experts and without identity experts")
        outputs = spec.n_experts + spec.n_identity
        if spec.scoring in ("top_softmax", "sigmoid"):
            if spec.n_identity or spec.groups != 1 or spec.route_scale != 1.0:
                raise ValueError("identity experts, groups and a scale of the weights belong to the scoring softmax_all")
        else:
            if spec.n_identity < 0 or outputs > 512 or spec.top > outputs:
                raise ValueError(f"the router has 1 to 512 outputs and a token takes at most all of them, not {spec.top} of {outputs}")
            if spec.groups < 1 or outputs % spec.groups or not 1 <= spec.groups_kept <= spec.groups:
                raise ValueError(f"{outputs} router outputs do not form {spec.groups} equal groups of which "
                                 f"{spec.groups_kept} are kept")
            if spec.shared_gate:
                raise ValueError("the gate of a shared expert is one more router row of the scoring top_softmax only")
        self.spec = spec
        self.dtype = dtype
        self.gated = spec.expert_act == "silu_gated"
        width, ff = spec.hidden_size, spec.expert_size
        self.router_rows = outputs + (1 if spec.shared_gate else 0)
        # stored in 16 bits it stays so: products of two bfloat16 numbers are exact in float32, and the
        # product kernels add them up in float32 and hand the sums back unrounded
        self.add_param("router", (self.router_rows, width), dtype, device)
        if spec.router_bias:
            self.add_param("router_bias", (outputs,), torch.float32, device, role="vector")
        # expert e: rows [e * 2 ff, e * 2 ff + ff) its gate, the next ff its up; rows [e * width, ...) its down
        # (plain experts: rows [e * ff, ...) its up)
        if self.gated:
            self.add_param("gate_up", (spec.n_experts * 2 * ff, width), dtype, device)
        else:
            self.add_param("up", (spec.n_experts * ff, width), dtype, device)
        self.add_param("down", (spec.n_experts * width, ff), dtype, device)
        if spec.shared_size is not None:
            element_size = torch.empty((), dtype=dtype).element_size()
            self.add_param("shared_gate_up", (2 * spec.shared_size, width), dtype, device,
                           row_padding=plan.gated_row_padding(width, element_size))
            self.add_param("shared_down", (width, spec.shared_size), dtype, device)

    def forward(self, h: torch.Tensor, ctx) -> torch.Tensor:
        spec = self.spec
        logits = ops.linear(h, self.params["router"], out_dtype=torch.float32)
        identity = None
        if spec.scoring == "softmax_all":
            shared_gate = None
            experts, weights, identity = ops.route_scored(
                logits, self.params.get("router_bias"), n_experts=spec.n_experts, top=spec.top, groups=spec.groups,
                keep=spec.groups_kept, scale=spec.route_scale)
        else:
            experts, weights, shared_gate = ops.route_top(
                logits, self.params.get("router_bias"), n_experts=spec.n_experts, top=spec.top,
                shared_gate=spec.shared_gate, scoring=spec.scoring)
        first = self.params["gate_up"] if self.gated else self.params["up"]
        shared = None
        if spec.shared_size is not None:
            shared_hidden = ops.linear_glu(h, self.params["shared_gate_up"], out_dtype=self.dtype)
            shared = ops.linear(shared_hidden, self.params["shared_down"], out_dtype=torch.float32)
        if h.shape[0] >= ops.GROUPED_FROM and ops.experts_grouped_ok(h, first, self.params["down"]):
            # many tokens: sorted by expert, every expert's tokens as tiles on the matrix cores
            return ops.experts_grouped(h, first, self.params["down"], experts, weights,
                                       n_experts=spec.n_experts, ff=spec.expert_size, shared=shared,
                                       shared_gate=shared_gate, act=spec.expert_act, identity_weight=identity,
                                       weight_on_input=spec.weight_on_input)
        hidden = ops.expert_gate_up(h, first, experts, n_experts=spec.n_experts, ff=spec.expert_size,
                                    act=spec.expert_act, input_weights=weights if spec.weight_on_input else None)
        if spec.weight_on_input:
            weights = torch.ones_like(weights)  # the weights went in with the inputs
        return ops.expert_down(hidden, self.params["down"], experts, weights, n_experts=spec.n_experts,
                               width=spec.hidden_size, shared=shared, shared_gate=shared_gate,
                               identity_x=h if identity is not None else None, identity_weight=identity)


register_part("feed_forward", "mixture", MixtureFeedForward, replace=True)
