"""What every part of a layer looks like to the model that assembles it.

A part owns named parameters (device tensors the weight loader fills by path) and a
``forward``.  It gets its sizes and constants from its spec and the batch from the
step context; it does not know which model, or which layer of it, it sits in.

Interfaces
----------
norm          ``forward(x) -> y`` and ``add_forward(resid, delta, row_idx=None) -> y``:
              ``resid`` is the float32 residual stream, ``delta`` the previous part's
              output (or None), either ``[tokens, dim]`` or a stack ``[parts, tokens, dim]``
              of float32 partial sums still to be added up (:func:`summed` makes one float32
              tensor of either), or a :class:`Normed` (such an output that is normed before it
              is added); the sum is formed in float32, stored back into
              ``resid`` (unless ``row_idx`` picks rows), and its norm is returned in
              the activation dtype.
position      ``rotary() -> (inv_freq, rotary_dim) | None`` for encodings applied by
              rotating q and k: float32 frequencies of the pairs ``(i, i + rotary_dim/2)``
              of the first ``rotary_dim`` elements of a head; None encodes nothing.
mixer         ``cache_requirement() -> KVRequirement | StateRequirement | a tuple of them | None`` and
              ``forward(h, ctx, cache, stores) -> [tokens, hidden]`` (or partial sums
              ``[parts, tokens, hidden]`` in float32, see norm): ``cache`` is the
              view of the run's cache (its own, or the one it borrows); ``stores``
              says whether this run writes it.
feed_forward  ``forward(h, ctx) -> [tokens, hidden]``.
block         ``forward(resid, delta, ctx, cache, stores) -> (resid, delta)``: takes and
              returns the residual stream and the not-yet-added output of the last part.
stream        ``forward(resid, ctx) -> resid``: the embedded tokens (float32 ``[tokens, dim]``)
              before the first layer: an embedding norm, learned positions
              (``ctx.positions``), a scale.
logits        ``forward(logits, ctx) -> logits``: float32 ``[wanted, vocab]`` after the
              vocabulary head: a soft cap, a scale, a bias (in place).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Iterator, Optional, Tuple

import torch


@dataclass(frozen=True)
class KVRequirement:
    """A growing cache of keys and values: one entry per token, in pages.

    Runs whose requirements are equal share a group of pages (one block table)."""

    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None  # keep only the last `window` tokens' entries
    v_head_dim: Optional[int] = None  # size of a value head where it differs from a key head's
    # keep only the entries of the chunk of `chunk` positions that the next token falls into
    # (chunks counted from the request's first token)
    chunk: Optional[int] = None
    # False: one entry per token only (a latent from which keys and values are both made);
    # no tensor of values is kept, and the run's view has ``v`` None
    values: bool = True

    @property
    def value_dim(self) -> int:
        if not self.values:
            return 0
        return self.head_dim if self.v_head_dim is None else self.v_head_dim

    @property
    def bounded(self) -> bool:
        """Whether a request needs only a bounded number of this cache's entries."""
        return self.window is not None or self.chunk is not None

    @property
    def span(self) -> Optional[int]:
        """The most entries a token ever looks back over, itself included (None: all)."""
        return self.window if self.window is not None else self.chunk

    def first_needed(self, length: int) -> int:
        """The first position that the token at position ``length`` (the next one of a request
        that holds ``length``) still sees."""
        if self.window is not None:
            return max(0, length - self.window + 1)
        if self.chunk is not None:
            return length // self.chunk * self.chunk
        return 0


@dataclass(frozen=True)
class StateRequirement:
    """Per-request state of fixed size, overwritten in place by every step.  A run that keeps
    several states (or one beside its keys and values) gives each a ``name``; the run's cache
    view then holds it as ``states[name]``."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32
    name: str = ""


def requirement_list(need) -> Tuple[object, ...]:
    """What a run keeps, as a tuple: ``cache_requirement()`` may return nothing, one
    requirement, or several (at most one of them keys and values)."""
    if need is None:
        return ()
    if isinstance(need, (KVRequirement, StateRequirement)):
        return (need,)
    return tuple(need)


@dataclass
class Normed:
    """A part's output that is still to be divided by its root mean square (``eps`` inside the
    root), multiplied by ``gain`` (one float32 number on the device) and added to the residual
    stream: what a layer that norms its sublayers on both sides hands to the next norm.
    ``value`` is ``[tokens, dim]`` or a stack ``[parts, tokens, dim]`` of float32 partial sums."""

    value: torch.Tensor
    gain: torch.Tensor
    eps: float


@dataclass
class Scaled:
    """A part's output that is still to get a ``bias`` per element (a projection's bias that was left
    for the sum), to be multiplied element by element by ``scale`` and added to the residual stream
    (either may be None).  ``value`` as in :class:`Normed`."""

    value: torch.Tensor
    scale: Optional[torch.Tensor] = None
    bias: Optional[torch.Tensor] = None


@dataclass
class DepthMixed(Scaled):
    """As :class:`Scaled`, and once it is added the sum is a layer's result: it becomes
    ``streams[index]`` (float32 ``[total, tokens, dim]``, one stream per layer so far and the embedded
    tokens first), and the residual stream is replaced by ``sum_{j <= index} coeff[j] * streams[j]``."""

    streams: Optional[torch.Tensor] = None
    index: int = 0
    coeff: Optional[torch.Tensor] = None


def summed(delta: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    """A part's output that has not been added to the residual stream yet, as one float32
    ``[tokens, dim]`` tensor.  What a mixer or a feed-forward hands on is either a tensor of
    that shape in the activation dtype or a stack ``[parts, tokens, dim]`` of float32 partial
    sums (the product kernels cut the reduction over workgroups for some row counts); which
    of the two depends on the step's size, so a norm or a block that adds it up itself goes
    through this function (the built-in norm kernel takes both forms directly)."""
    if delta is None:
        return None
    if isinstance(delta, Normed):
        value = summed(delta.value)
        rms = torch.sqrt(value.square().mean(dim=-1, keepdim=True) + delta.eps)
        return value / rms * delta.gain.float()
    if isinstance(delta, DepthMixed):
        raise TypeError("a layer's result that is mixed with the earlier layers' needs a norm that knows how "
                        "(the built-in rmsnorm does)")
    if isinstance(delta, Scaled):
        value = summed(delta.value)
        if delta.bias is not None:
            value = value + delta.bias.float()
        return value if delta.scale is None else value * delta.scale.float()
    return delta.sum(dim=0) if delta.dim() == 3 else delta.float()


class Part:
    """Base of all parts: a bag of named parameters and named sub-parts."""

    def __init__(self) -> None:
        self.params: Dict[str, torch.Tensor] = {}
        self.param_roles: Dict[str, str] = {}
        self.children: Dict[str, "Part"] = {}

    def add_param(self, name: str, shape, dtype: torch.dtype, device, role: str = "matrix",
                  row_padding: int = 0) -> None:
        """``row_padding``: elements left unused behind every row of a matrix in memory; the
        parameter is then the view of its rows without them, with a row stride of its own."""
        shape = tuple(shape)
        if row_padding and len(shape) == 2:
            self.params[name] = torch.empty((shape[0], shape[1] + row_padding), dtype=dtype,
                                            device=device)[:, : shape[1]]
        else:
            self.params[name] = torch.empty(shape, dtype=dtype, device=device)
        self.param_roles[name] = role

    def add_child(self, name: str, part: "Part") -> "Part":
        self.children[name] = part
        return part

    def named_params(self, prefix: str = "") -> Iterator[Tuple[str, "Part", str]]:
        """``(path, owner, name)`` of every parameter below this part."""
        for name in self.params:
            yield prefix + name, self, name
        for child_name, child in self.children.items():
            yield from child.named_params(prefix + child_name + ".")
