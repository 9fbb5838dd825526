"""The arrangement of a layer's parts.  ``pre_norm``
(/root/reference/src/pylon/model/layers.py:176-200):
``x = x + mixer(norm1(x)); x = x + feed_forward(norm2(x))``.

The residual stream is float32.  A block receives the stream together with the
previous part's output that has not been added yet, so that every residual sum is
formed inside the norm kernel that follows it; it hands back the same pair.

A ``pre_norm`` layer may also have: a short convolution or a token shift on ``norm1``'s output
(``input_conv``; the norm's output then stays float32 until the shift has rounded it once); a learned
scale per element on each sublayer's output (``sublayer_scale``); a feed-forward or mixer that leaves
its output projection's bias to the sum (``output_bias``); and ``depth_mix``: the layer's result is kept
as one of the streams of the step, and what it hands on is a learned mix of all streams so far.  All of
these travel to the next norm as :class:`~.base.Scaled` or :class:`~.base.DepthMixed` and cost no launch
of their own."""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from ..config.specs import LayerSpec
from .base import DepthMixed, Part, Scaled, requirement_list
from .registry import build_part, register_part


class PreNormBlock(Part):
    def __init__(self, spec: LayerSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        self.spec = spec
        self.dtype = dtype
        kw = dict(dtype=dtype, device=device)
        self.input_conv = None
        if spec.input_conv is not None:
            self.input_conv = self.add_child("input_conv", build_part("conv", spec.input_conv, **kw))
        self.mixer_norm = self.add_child("mixer_norm", build_part(
            "norm", spec.mixer_norm, dtype=torch.float32 if self.input_conv is not None else dtype, device=device))
        self.mixer = self.add_child("mixer", build_part("mixer", spec.mixer, **kw))
        if (spec.feed_forward is None) != (spec.feed_forward_norm is None):
            raise ValueError("a feed-forward and its norm come together or not at all")
        self.feed_forward = None  # a layer may consist of its mixer alone
        if spec.feed_forward is not None:
            self.feed_forward_norm = self.add_child(
                "feed_forward_norm", build_part("norm", spec.feed_forward_norm, **kw)
            )
            self.feed_forward = self.add_child(
                "feed_forward", build_part("feed_forward", spec.feed_forward, **kw)
            )
        width = spec.mixer_norm.dim
        if spec.sublayer_scale:
            self.add_param("mixer_scale", (width,), torch.float32, device, role="vector")
            if self.feed_forward is not None:
                self.add_param("feed_forward_scale", (width,), torch.float32, device, role="vector")
        if spec.depth_mix is not None:
            index, total = spec.depth_mix
            if not 1 <= index < total:
                raise ValueError(f"a layer's result is stream 1 to {total - 1} of {total}, not {index}")
            self.add_param("depth_coeff", (index + 1,), torch.float32, device, role="vector")
        # a sublayer that can leave its last bias to the residual sum is told to
        for part in (self.mixer, self.feed_forward):
            if part is not None and hasattr(part, "defer_output_bias"):
                part.defer_output_bias = True

    def cache_requirement(self):
        needs = requirement_list(self.mixer.cache_requirement())
        if self.input_conv is not None:
            needs += requirement_list(self.input_conv.cache_requirement())
        return None if not needs else (needs[0] if len(needs) == 1 else needs)

    def decode_signature(self, rows: int, bound: int) -> tuple:
        describe = getattr(self.mixer, "decode_signature", None)
        return ("bound", bound) if describe is None else describe(rows, bound)

    def forward(self, resid: torch.Tensor, delta: Optional[torch.Tensor], ctx, cache,
                stores: bool) -> Tuple[torch.Tensor, torch.Tensor]:
        h = self.mixer_norm.add_forward(resid, delta)
        streams = None
        if self.spec.depth_mix is not None:
            # the step's streams, shared by its layers: the first layer that mixes makes them and
            # puts in what it was handed (the embedded tokens) as stream 0
            streams = ctx.memo.get("depth_streams")
            if streams is None:
                streams = torch.empty((self.spec.depth_mix[1], *resid.shape), dtype=torch.float32, device=resid.device)
                streams[0].copy_(resid)
                ctx.memo["depth_streams"] = streams
        if self.input_conv is not None:
            h = self.input_conv.forward(h, ctx, cache)
        mixed = self._pending(self.mixer, self.mixer.forward(h, ctx, cache, stores), "mixer_scale")
        if self.feed_forward is None:
            return resid, self._result(mixed, streams)
        h = self.feed_forward_norm.add_forward(resid, mixed)
        out = self._pending(self.feed_forward, self.feed_forward.forward(h, ctx), "feed_forward_scale")
        return resid, self._result(out, streams)

    def _pending(self, part, value, scale_name: str):
        """A sublayer's output with what is still to happen to it on its way into the sum."""
        scale = self.params.get(scale_name)
        bias = getattr(part, "output_bias", None) if getattr(part, "defer_output_bias", False) else None
        if scale is None and bias is None:
            return value
        return Scaled(value, scale, bias)

    def _result(self, pending, streams):
        """The layer's last output: as it is, or to be mixed with the earlier layers' results."""
        if streams is None:
            return pending
        if not isinstance(pending, Scaled):
            pending = Scaled(pending)
        return DepthMixed(pending.value, pending.scale, pending.bias, streams=streams,
                          index=self.spec.depth_mix[0], coeff=self.params["depth_coeff"])


class SandwichNormBlock(Part):
    """Every sublayer normed on both sides: ``x += post1(mixer(conv(norm1(x))))``, then, if the
    layer has a feed-forward, ``x += post2(ff(norm2(x)))``; ``conv`` is an optional short
    convolution in front of the mixer, whose input is then kept in float32.  The norm after a
    sublayer is not a launch of its own: its output travels as :class:`~.base.Normed` to the
    next norm, which norms it, adds it and norms the sum in one kernel."""

    def __init__(self, spec: LayerSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        if spec.mixer_post_norm is None:
            raise ValueError("a sandwich_norm layer needs the norm after its mixer")
        if (spec.feed_forward is None) != (spec.feed_forward_norm is None) or \
                (spec.feed_forward is None) != (spec.feed_forward_post_norm is None):
            raise ValueError("a feed-forward and its two norms come together or not at all")
        self.spec = spec
        kw = dict(dtype=dtype, device=device)
        self.input_conv = None
        if spec.input_conv is not None:
            self.input_conv = self.add_child("input_conv", build_part("conv", spec.input_conv, **kw))
        self.mixer_norm = self.add_child("mixer_norm", build_part(
            "norm", spec.mixer_norm, dtype=torch.float32 if self.input_conv is not None else dtype, device=device))
        self.mixer = self.add_child("mixer", build_part("mixer", spec.mixer, **kw))
        self.mixer_post_norm = self.add_child("mixer_post_norm", build_part("norm", spec.mixer_post_norm, **kw))
        self.feed_forward = None
        if spec.feed_forward is not None:
            self.feed_forward_norm = self.add_child("feed_forward_norm", build_part("norm", spec.feed_forward_norm, **kw))
            self.feed_forward = self.add_child("feed_forward", build_part("feed_forward", spec.feed_forward, **kw))
            self.feed_forward_post_norm = self.add_child(
                "feed_forward_post_norm", build_part("norm", spec.feed_forward_post_norm, **kw))

    def cache_requirement(self):
        needs = requirement_list(self.mixer.cache_requirement())
        if self.input_conv is not None:
            needs += requirement_list(self.input_conv.cache_requirement())
        return needs if len(needs) != 1 else needs[0]

    def decode_signature(self, rows: int, bound: int) -> tuple:
        describe = getattr(self.mixer, "decode_signature", None)
        return ("bound", bound) if describe is None else describe(rows, bound)

    def forward(self, resid: torch.Tensor, delta, ctx, cache, stores: bool):
        h = self.mixer_norm.add_forward(resid, delta)
        if self.input_conv is not None:
            h = self.input_conv.forward(h, ctx, cache)
        pending = self.mixer_post_norm.pending(self.mixer.forward(h, ctx, cache, stores))
        if self.feed_forward is None:
            return resid, pending
        h = self.feed_forward_norm.add_forward(resid, pending)
        return resid, self.feed_forward_post_norm.pending(self.feed_forward.forward(h, ctx))


register_part("block", "pre_norm", PreNormBlock, replace=True)
register_part("block", "sandwich_norm", SandwichNormBlock, replace=True)
