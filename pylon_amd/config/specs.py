"""Typed descriptions of the parts a decoder is assembled from.

A model is data: a tuple of :class:`LayerSpec` (what each layer is made of) and a
tuple of :class:`ScheduleEntry` (in which order layers run and whose cache each
run uses).  Every size and constant a part needs is a field of its spec; the
parts never look at an architecture's config.json themselves.

The specs mirror what the reference hard-codes per block
(/root/reference/src/pylon/model/layers.py:81-108 attention sizes,
:13-27 feed-forward sizes, :30-40 norm eps, :43-51 rotary constants).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Tuple


@dataclass(frozen=True)
class NormSpec:
    """A normalisation over the last axis of ``dim`` elements."""

    kind: str
    dim: int
    eps: float
    # what is added to the stored weight before it multiplies: 1.0 for weights stored around zero
    weight_offset: float = 0.0


@dataclass(frozen=True)
class RotaryScalingSpec:
    """Frequencies stretched for contexts longer than the ``original`` one: with ``where(t) =
    rotary_dim * ln(original / (2 pi t)) / (2 ln theta)`` the (fractional) pair that makes ``t`` turns
    over the original length, ``lo = max(floor(where(fast)), 0)``, ``hi = min(ceil(where(slow)),
    rotary_dim - 1)`` and ``ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1)``, pair ``i`` turns
    at ``f_i / factor * ramp_i + f_i * (1 - ramp_i)``, and every cosine and sine is multiplied by
    ``0.1 * ln(factor) + 1``."""

    factor: float
    original: float
    fast: float
    slow: float


@dataclass(frozen=True)
class PositionSpec:
    """How positions enter a mixer.

    ``kind="rope"``: rotate the first ``rotary_dim`` elements of every head by
    ``position * theta**(-2i/rotary_dim)``, pairing element ``i`` with
    ``i + rotary_dim/2``.  ``kind="none"``: positions are not encoded.
    ``scaling``: see :class:`RotaryScalingSpec`.
    """

    kind: str
    theta: float = 10000.0
    rotary_dim: int = 0
    max_positions: int = 0
    # True: element 2i turns together with its neighbour 2i + 1 instead of with i + rotary_dim/2
    interleaved: bool = False
    scaling: Optional[RotaryScalingSpec] = None


@dataclass(frozen=True)
class AttentionSpec:
    """Grouped-query softmax attention over a paged key/value cache."""

    hidden_size: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    scale: float
    position: PositionSpec
    qk_norm: bool = False
    qk_norm_eps: float = 1e-6
    window: Optional[int] = None  # None: every earlier key; w: the last w keys
    kind: str = "attention"
    # "head": q and k are normed head by head, weights of head_dim elements; "projection": one
    # norm over all heads of q at once and one over all heads of k, weights of the projections' sizes
    qk_norm_over: str = "head"
    v_head_dim: Optional[int] = None  # size of a value head where it differs from a key head's
    # c: position i sees key j <= i only if floor(i / c) == floor(j / c), chunks counted from the
    # request's first token (not together with a window)
    chunk: Optional[int] = None
    # the scaled score s becomes softcap * tanh(s / softcap)
    softcap: Optional[float] = None
    # True: a learned number per head joins the softmax's denominator as exp(sink_h): a key without
    # a value whose score is neither scaled nor capped
    sink: bool = False
    # "head": every head's output is multiplied by sigmoid(W_g h) of that head (W_g has one row a
    # head); "element": the concatenated heads element by element (one row an element); both read
    # the mixer's input, as the projections do
    output_gate: Optional[str] = None
    # True: there is no value projection; the values are the keys as projected, before their norm
    # and rotation
    values_from_keys: bool = False

    @property
    def q_size(self) -> int:
        return self.n_heads * self.head_dim

    @property
    def gate_size(self) -> int:
        """Rows of the gate's projection."""
        if self.output_gate is None:
            return 0
        return self.n_heads if self.output_gate == "head" else self.n_heads * self.value_dim

    @property
    def kv_size(self) -> int:
        return self.n_kv_heads * self.head_dim

    @property
    def value_dim(self) -> int:
        return self.head_dim if self.v_head_dim is None else self.v_head_dim

    @property
    def v_size(self) -> int:
        return self.n_kv_heads * self.value_dim


@dataclass(frozen=True)
class SinkAttentionSpec:
    """Grouped-query softmax attention without rotation: positions enter as a learned bias by
    distance, and the softmax has a sink (a key of score 0 without a value: one is added to the
    denominator).  ``score = scale * q.k + rel[bucket(i - j), head]`` with ``bias_rows`` rows in
    ``rel``: distances below ``bias_rows // 2`` have a row each, the other half of the rows
    spreads logarithmically up to ``bias_far``, beyond which the last row is used.  Keys have
    ``head_dim`` elements, values ``v_head_dim``.

    ``bias_form="log"`` replaces the table by two learned numbers per head, ``a`` and ``b``:
    ``score = scale * q.k - a * log(1 + b * (i - j))`` (``bias_rows`` and ``bias_far`` are then
    unused).  ``chunk``: position ``i`` sees key ``j <= i`` only inside its own chunk of that many
    positions (as in :class:`AttentionSpec`; not together with a window).  ``qkv_bias``: the q, k and v
    projections have a bias each.  ``own_kv`` False: a layer that only ever runs on another run's keys
    and values and has no k and v projections of its own."""

    hidden_size: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    v_head_dim: int
    scale: float
    bias_rows: int
    bias_far: float
    sink: bool = True
    window: Optional[int] = None
    kind: str = "sink_attention"
    bias_form: str = "table"
    chunk: Optional[int] = None
    qkv_bias: bool = False
    own_kv: bool = True
    # False: the cache keeps every token's keys and values although the layer's own mask would let
    # old pages go (runs with other masks read the same cache)
    cache_bounded: bool = True


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Softmax attention whose keys and values are made from one small latent per token, the only
    thing cached: ``c = norm(W_dkv h)`` (``kv_rank`` numbers), per head ``k = W_uk c``,
    ``v = W_uv c``; queries through a latent of their own, ``q = W_uq norm(W_dq h)``; no
    positions; ``score = scale * q.k`` over a sliding ``window`` (None: every earlier key), a
    ``chunk`` (as in :class:`AttentionSpec`) or everything before; with ``gate`` every head's
    output is multiplied by ``sigmoid(W_g h)`` of that head before the output projection.  The
    latents' norms divide by the root mean square (``norm_eps`` inside the root) and multiply by a
    weight."""

    hidden_size: int
    n_heads: int
    head_dim: int
    v_head_dim: int
    q_rank: int
    kv_rank: int
    scale: float
    norm_eps: float
    window: Optional[int] = None
    chunk: Optional[int] = None
    gate: bool = True
    kind: str = "latent_attention"


@dataclass(frozen=True)
class RetentionSpec:
    """Linear attention with one fixed decay per head and no softmax:
    ``S_t = decay_h S_{t-1} + k_t v_t^T``, ``o_t = S_t^T q_t``; q and k are rotated by
    ``position`` (k then multiplied by ``head_dim ** -0.5``), every head's ``o`` is divided by
    its root mean square (``norm_eps`` inside the root), the heads are multiplied by
    ``silu(W_g h)`` and projected."""

    hidden_size: int
    n_heads: int
    head_dim: int
    v_head_dim: int
    decay: Tuple[float, ...]
    position: PositionSpec
    norm_eps: float
    kind: str = "retention"


@dataclass(frozen=True)
class DeltaRuleSpec:
    """The gated delta rule: per request and head a float32 state ``S`` of ``head_dim x v_head_dim``,
    ``S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q`` (the read-out sees the token's own
    write).  ``q`` and ``k`` have ``n_kv_heads`` heads (head ``h`` uses ``h // (n_heads / n_kv_heads)``),
    ``v`` has ``n_heads``; each of the three passes a causal convolution of ``conv_taps`` taps per
    channel and ``silu``; q and k become unit vectors per head (``unit_eps`` inside the root), q also
    times ``head_dim ** -0.5``; ``beta = sigmoid(W_b h)``, ``g = exp(-exp(A_log) * softplus(W_a h +
    dt_bias))`` per head; every head's ``o`` is divided by its root mean square (``norm_eps``), times a
    weight shared by the heads, times ``silu(W_g h)``; then the output projection."""

    hidden_size: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    v_head_dim: int
    conv_taps: int
    norm_eps: float
    unit_eps: float = 1e-6
    kind: str = "delta_rule"


@dataclass(frozen=True)
class ParallelMixerSpec:
    """Two mixers side by side on the same input: ``left_scale * left(h) + right_scale * right(h)``;
    ``left`` and ``right`` are mixer specs of any kind (at most one of them keeps keys and values)."""

    left: object
    right: object
    left_scale: float = 1.0
    right_scale: float = 1.0
    kind: str = "parallel"


@dataclass(frozen=True)
class TokenShiftSpec:
    """``h + (h' - h) * w``: every token's input moved towards the previous token's (``h'``, zeros
    before a request's first token) by a learned share per channel; a request's last input is its
    state."""

    dim: int
    kind: str = "token_shift"


@dataclass(frozen=True)
class SinusoidPositionSpec:
    """A fixed position vector added to the embedded tokens: element ``2i`` is
    ``sin(p * base**(-2i/dim))``, element ``2i + 1`` the cosine of the same angle."""

    dim: int
    base: float = 10000.0
    kind: str = "sinusoid"


@dataclass(frozen=True)
class ShortConvSpec:
    """``h + conv(h)``: a causal convolution of ``taps`` taps over time on each of ``dim``
    channels, added to its input; a request's last ``taps - 1`` inputs are its state."""

    dim: int
    taps: int
    kind: str = "short_conv"


@dataclass(frozen=True)
class CappedGatedFeedForwardSpec:
    """``down(a(g) * (u + offset))`` with ``g = min(gate(x), limit)``, ``u = clamp(up(x), -limit,
    limit)`` and ``a(g) = g * sigmoid(alpha * g)``; gate and up fused into one matrix."""

    hidden_size: int
    intermediate_size: int
    limit: float
    alpha: float = 1.702
    offset: float = 1.0
    kind: str = "capped_gated_mlp"


@dataclass(frozen=True)
class MixtureFeedForwardSpec:
    """A mixture of ``n_experts`` gated feed-forwards of ``expert_size`` hidden units, of which
    every token uses the ``top`` with the largest router logits ``W_r h + b`` (float32), weighted
    by the softmax over those ``top`` logits alone; an expert is ``down(silu(gate(h)) * up(h))``.
    With ``shared_size`` a further expert of that many hidden units runs for every token and is
    added, multiplied by ``sigmoid(w_sg . h)`` if ``shared_gate``.

    ``expert_act="relu2"``: plain experts, ``down(relu(up(h))^2)``.  ``scoring="softmax_all"``: the
    scores are the softmax over all router outputs; the ``router_bias`` is a correction added to
    them for the choice only; the router's outputs form ``groups`` equal groups of neighbours of
    which only the ``groups_kept`` with the largest corrected score can be chosen from; the weights
    are the chosen scores times ``route_scale``, not renormalised.  The router's last ``n_identity``
    outputs (beyond the ``n_experts`` experts, and counted in the groups) are identity experts whose
    output is the input itself.

    ``scoring="sigmoid"``: the scores are the sigmoids of the router's outputs, the ``top`` largest
    are chosen and their scores are the weights as they are.  ``weight_on_input``: a chosen expert's
    weight multiplies its input instead of its output, ``sum_e expert_e(w_e h)``."""

    hidden_size: int
    n_experts: int
    top: int
    expert_size: int
    shared_size: Optional[int] = None
    shared_gate: bool = True
    router_bias: bool = True
    kind: str = "mixture"
    expert_act: str = "silu_gated"
    scoring: str = "top_softmax"
    n_identity: int = 0
    groups: int = 1
    groups_kept: int = 1
    route_scale: float = 1.0
    weight_on_input: bool = False


@dataclass(frozen=True)
class LogitSoftcapSpec:
    """``logits <- cap * tanh(logits / cap)``."""

    cap: float
    kind: str = "softcap"


@dataclass(frozen=True)
class LogitScaleSpec:
    """Logits times one constant."""

    factor: float
    kind: str = "scale"


@dataclass(frozen=True)
class GatedFeedForwardSpec:
    """``down(act(gate(x)) * up(x))`` with gate and up fused into one matrix; with ``bias`` all
    three projections have one."""

    hidden_size: int
    intermediate_size: int
    activation: str = "silu"
    kind: str = "gated_mlp"
    bias: bool = False


@dataclass(frozen=True)
class LayerSpec:
    """One residual block: which mixer, which feed-forward, which norms, how arranged.

    ``arrangement="pre_norm"``: ``x += mixer(norm1(x)); x += ff(norm2(x))``.
    ``arrangement="sandwich_norm"``: every sublayer is normed on both sides,
    ``x += post1(mixer(conv(norm1(x)))); x += post2(ff(norm2(x)))``, where ``conv`` is the
    optional ``input_conv`` in front of the mixer and ``feed_forward`` may be None.

    In the ``pre_norm`` arrangement: ``input_conv`` (a short convolution or a token shift) works on
    ``norm1``'s output; with ``sublayer_scale`` each sublayer's output is multiplied element by element
    by a learned vector before it is added; ``depth_mix = (index, total)`` makes the layer's result
    stream ``index`` of ``total`` (stream 0: the embedded tokens) and hands on, instead of it, a learned
    mix ``sum_{j <= index} c[j] * stream_j`` of all streams so far.
    """

    mixer: object
    feed_forward: object
    mixer_norm: NormSpec
    feed_forward_norm: Optional[NormSpec]
    arrangement: str = "pre_norm"
    mixer_post_norm: Optional[NormSpec] = None
    feed_forward_post_norm: Optional[NormSpec] = None
    input_conv: Optional[object] = None
    sublayer_scale: bool = False
    depth_mix: Optional[Tuple[int, int]] = None

    @property
    def kind(self) -> str:
        return self.arrangement


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer.

    ``layer`` indexes :attr:`ModelSpec.layers`; a layer may be named by several
    entries and then runs again with the same weights.  ``cache`` names the
    cache this run works on: by default its own (the index of the entry in the
    schedule).  An entry whose ``cache`` is an *earlier* entry's index reads
    that entry's keys and values and stores none of its own.
    """

    layer: int
    cache: Optional[int] = None
    # True: the embedded tokens (the stream as it was before the first run) are added to the
    # stream once more right before this run
    add_embedding: bool = False


@dataclass(frozen=True)
class ModelSpec:
    vocab_size: int
    hidden_size: int
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[ScheduleEntry, ...]
    final_norm: NormSpec
    tie_word_embeddings: bool
    max_positions: int
    embedding_scale: float = 1.0
    # Parts between the embedding and the first layer (family "stream": an embedding norm,
    # learned positions, ...) and parts after the vocabulary head (family "logits": a soft
    # cap, a scale, ...), as specs with a ``kind``; the Qwen3 decoder has neither.
    stream_parts: Tuple[object, ...] = ()
    logit_parts: Tuple[object, ...] = ()
    extra: dict = field(default_factory=dict, compare=False, hash=False)

    def resolved_schedule(self) -> Tuple[Tuple[int, int, bool], ...]:
        """``(layer, cache_id, stores)`` per run, with defaults filled in and checked."""
        out = []
        for index, entry in enumerate(self.schedule):
            if not 0 <= entry.layer < len(self.layers):
                raise ValueError(
                    f"schedule entry {index} names layer {entry.layer}, "
                    f"but the model has {len(self.layers)} layers"
                )
            cache = index if entry.cache is None else entry.cache
            if cache > index or cache < 0:
                raise ValueError(
                    f"schedule entry {index} reads cache {cache}; a run may only "
                    "read its own cache or that of an earlier run"
                )
            if cache != index and out[cache][1] != cache:
                raise ValueError(
                    f"schedule entry {index} reads cache {cache}, which itself "
                    "borrows another run's cache"
                )
            out.append((entry.layer, cache, cache == index))
        return tuple(out)

    def embedding_again(self) -> Tuple[bool, ...]:
        """Per run: whether the embedded tokens are added to the stream before it."""
        return tuple(entry.add_embedding for entry in self.schedule)
