"""Gimudra: config.json keys, the model as specs, and checkpoint tensor names.

A decoder whose layers are listed one by one in ``layers``; each entry has a ``type`` (the mixer:
"attention"), the mixer's sizes under ``mixer`` and its feed-forward under ``mlp`` (null: none).

* The embedded tokens are multiplied by ``embedding.scale`` and get a sinusoidal position vector.
* A layer is pre-normed (RMS norms with ``norm.eps``).  What the mixer reads is first moved towards
  the previous token's input by a learned share per channel (``shift``); each sublayer's output is
  multiplied element by element by a learned vector (``ls1``, ``ls2``) before it is added; and what a
  layer hands on is not its result but a learned mix (``dwa``) of the embedded tokens and all layers'
  results so far.
* Attention: grouped queries, biases on the q, k and v projections, no rotation; from the scaled score
  (``scale`` from the config) ``r1_h * log(1 + r2_h * (i - j))`` is taken off; position ``i`` sees key
  ``j <= i`` only inside its own chunk of ``mask.size`` positions; values of ``vdim`` elements.  A mixer
  with ``kv_from: j`` has no k and v projections and attends over layer ``j``'s keys and values.
* Feed-forward "dense": ``W_down (silu(W_gate h) * W_up h)``, all three with biases.  "moe": ``experts``
  plain experts ``W_down relu(W_up h)^2`` and ``identity`` identity experts (their output is ``h``); scores
  are the softmax over all router outputs; ``correction`` is added for the choice only; the outputs form
  ``groups.count`` equal groups of neighbours of which the best ``groups.keep`` can be chosen from; a token
  takes ``top``; the weights are the chosen scores times ``router.scale``.
* The final norm, then the head (a matrix of its own).

Tensors: ``embed``, ``head``, ``final.norm``, per layer ``l<i>.norm1``, ``.norm2``, ``.ls1``, ``.ls2``,
``.shift``, ``.dwa``; attention ``.mix.{q,k,v}`` with ``.b``, ``.mix.o``, ``.mix.r1``, ``.mix.r2``; dense
``.mlp.{gate,up,down}`` with ``.b``; mixture ``.mlp.e<j>.{up,down}``, ``.mlp.router``, ``.mlp.correction``.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, Mapping, Optional, Tuple

from ..config.registry import Architecture, WeightTarget, register_architecture
from ..config.specs import (
    GatedFeedForwardSpec,
    LayerSpec,
    MixtureFeedForwardSpec,
    ModelSpec,
    NormSpec,
    ScheduleEntry,
    SinkAttentionSpec,
    SinusoidPositionSpec,
    TokenShiftSpec,
)

ARCHITECTURE = "Gimudra"

POSITION_BASE = 10000.0  # of the sinusoidal position vector


def _positive_int(value, name: str) -> int:
    if isinstance(value, bool) or not isinstance(value, int) or value < 1:
        raise ValueError(f"{name} must be a positive integer, got {value!r}")
    return value


def _count(value, name: str) -> int:
    if isinstance(value, bool) or not isinstance(value, int) or value < 0:
        raise ValueError(f"{name} must be a non-negative integer, got {value!r}")
    return value


def _positive(value, name: str) -> float:
    value = float(value)
    if not (value > 0 and math.isfinite(value)):
        raise ValueError(f"{name} must be positive and finite, got {value!r}")
    return value


def _require(data: Mapping, keys, where: str) -> None:
    missing = [key for key in keys if key not in data]
    if missing:
        raise ValueError(f"config.json lacks required keys in {where}: " + ", ".join(missing))


@dataclass(frozen=True)
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    mask_size: Optional[int]
    kv_from: Optional[int]


@dataclass(frozen=True)
class DenseConfig:
    ff: int


@dataclass(frozen=True)
class MixtureConfig:
    experts: int
    identity: int
    top: int
    ff: int
    groups: int
    groups_kept: int
    scale: float


@dataclass(frozen=True)
class LayerConfig:
    type: str
    mixer: AttentionConfig
    mlp: Optional[object]  # DenseConfig, MixtureConfig or None


@dataclass(frozen=True)
class GimudraConfig:
    vocab: int
    width: int
    layers: Tuple[LayerConfig, ...]
    norm_eps: float
    embedding_scale: float
    initializer_range: float = 0.02  # only used to draw random weights
    eos_token_id: Optional[Tuple[int, ...]] = None


def _parse_mixer(kind: str, m: Mapping, where: str, index: int) -> AttentionConfig:
    if kind != "attention":
        raise ValueError(f"{where}: unknown layer type {kind!r} (known: attention)")
    _require(m, ("heads", "kv_heads", "dim", "vdim", "scale"), where)
    heads, kv_heads = _positive_int(m["heads"], "heads"), _positive_int(m["kv_heads"], "kv_heads")
    if heads % kv_heads:
        raise ValueError("The number of Q heads must be divisible by the number of KV heads.")
    mask = m.get("mask")
    size = None
    if mask is not None:
        _require(mask, ("size",), where + ".mask")
        size = _positive_int(mask["size"], "mask.size")
    kv_from = m.get("kv_from")
    if kv_from is not None:
        kv_from = _count(kv_from, "kv_from")
        if kv_from >= index:
            raise ValueError(f"{where}: kv_from {kv_from} must name an earlier layer")
    return AttentionConfig(heads, kv_heads, _positive_int(m["dim"], "dim"), _positive_int(m["vdim"], "vdim"),
                           _positive(m["scale"], "scale"), size, kv_from)


def _parse_mlp(mlp: Optional[Mapping], where: str):
    if mlp is None:
        return None
    _require(mlp, ("kind",), where)
    if mlp["kind"] == "dense":
        _require(mlp, ("ff",), where)
        return DenseConfig(_positive_int(mlp["ff"], "ff"))
    if mlp["kind"] != "moe":
        raise ValueError(f"{where}: unknown feed-forward kind {mlp['kind']!r} (known: dense, moe)")
    _require(mlp, ("expert", "router"), where)
    _require(mlp["expert"], ("ff",), where + ".expert")
    router = mlp["router"]
    _require(router, ("experts", "top"), where + ".router")
    experts, top = _positive_int(router["experts"], "experts"), _positive_int(router["top"], "top")
    identity = _count(router.get("identity", 0), "identity")
    outputs = experts + identity
    if top > outputs:
        raise ValueError(f"{where}: top {top} exceeds the {outputs} router outputs")
    groups = router.get("groups")
    count, keep = 1, 1
    if groups is not None:
        _require(groups, ("count", "keep"), where + ".router.groups")
        count, keep = _positive_int(groups["count"], "groups.count"), _positive_int(groups["keep"], "groups.keep")
        if outputs % count or keep > count:
            raise ValueError(f"{where}: {outputs} router outputs do not form {count} equal groups of which {keep} are kept")
    return MixtureConfig(experts, identity, top, _positive_int(mlp["expert"]["ff"], "expert.ff"), count, keep,
                         float(router.get("scale", 1.0)))


def parse_config(data: Mapping) -> GimudraConfig:
    _require(data, ("vocab", "width", "layers", "norm"), "the model")
    _require(data["norm"], ("eps",), "norm")
    layers = []
    for index, entry in enumerate(data["layers"]):
        where = f"layers[{index}]"
        _require(entry, ("type", "mixer"), where)
        layers.append(LayerConfig(entry["type"], _parse_mixer(entry["type"], entry["mixer"], where, index),
                                  _parse_mlp(entry.get("mlp"), where + ".mlp")))
    if not layers:
        raise ValueError("the model has no layers")
    for index, layer in enumerate(layers):
        source = layer.mixer.kv_from
        if source is None:
            continue
        lender, m = layers[source].mixer, layer.mixer
        if lender.kv_from is not None:
            raise ValueError(f"layers[{index}]: kv_from {source} names a layer that has no keys and values of its own")
        if (lender.kv_heads, lender.dim, lender.vdim, lender.heads) != (m.kv_heads, m.dim, m.vdim, m.heads):
            raise ValueError(f"layers[{index}]: its heads differ from those of layer {source}, whose keys and values it uses")
    embedding = data.get("embedding") or {}
    eos = data.get("eos_token_id")
    if isinstance(eos, int):
        eos = (eos,)
    elif eos is not None:
        eos = tuple(int(v) for v in eos)
    return GimudraConfig(
        vocab=_positive_int(data["vocab"], "vocab"), width=_positive_int(data["width"], "width"),
        layers=tuple(layers), norm_eps=_positive(data["norm"]["eps"], "norm.eps"),
        embedding_scale=float(embedding.get("scale", 1.0)),
        initializer_range=float(data.get("initializer_range", 0.02)), eos_token_id=eos)


def config_to_json(cfg: GimudraConfig) -> dict:
    layers = []
    for layer in cfg.layers:
        m = layer.mixer
        mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale}
        if m.mask_size is not None:
            mixer["mask"] = {"size": m.mask_size}
        if m.kv_from is not None:
            mixer["kv_from"] = m.kv_from
        mlp = None
        if isinstance(layer.mlp, DenseConfig):
            mlp = {"kind": "dense", "ff": layer.mlp.ff}
        elif layer.mlp is not None:
            f = layer.mlp
            mlp = {"kind": "moe", "expert": {"ff": f.ff},
                   "router": {"experts": f.experts, "identity": f.identity, "top": f.top, "scale": f.scale,
                              "groups": {"count": f.groups, "keep": f.groups_kept}}}
        layers.append({"type": layer.type, "mixer": mixer, "mlp": mlp})
    out = {"architecture": ARCHITECTURE, "vocab": cfg.vocab, "width": cfg.width, "layers": layers,
           "norm": {"eps": cfg.norm_eps}, "embedding": {"scale": cfg.embedding_scale},
           "initializer_range": cfg.initializer_range}
    if cfg.eos_token_id is not None:
        out["eos_token_id"] = list(cfg.eos_token_id)
    return out


def model_spec(cfg: GimudraConfig) -> ModelSpec:
    norm = NormSpec(kind="rmsnorm", dim=cfg.width, eps=cfg.norm_eps)
    total = len(cfg.layers) + 1  # streams of the depth mix: the embedded tokens and every layer's result
    layers, schedule = [], []
    # Layers that read one cache with different masks: that cache keeps every token (a cache whose
    # readers all have the same chunks lets the pages go that the chunk has left behind).
    masks: Dict[int, set] = {}
    for index, layer in enumerate(cfg.layers):
        owner = index if layer.mixer.kv_from is None else layer.mixer.kv_from
        masks.setdefault(owner, set()).add(layer.mixer.mask_size)
    for index, layer in enumerate(cfg.layers):
        m = layer.mixer
        owner = index if m.kv_from is None else m.kv_from
        mixer = SinkAttentionSpec(
            hidden_size=cfg.width, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim, v_head_dim=m.vdim,
            scale=m.scale, bias_rows=0, bias_far=0.0, sink=False, bias_form="log", chunk=m.mask_size, qkv_bias=True,
            own_kv=m.kv_from is None, cache_bounded=len(masks[owner]) == 1)
        feed_forward = None
        if isinstance(layer.mlp, DenseConfig):
            feed_forward = GatedFeedForwardSpec(hidden_size=cfg.width, intermediate_size=layer.mlp.ff, bias=True)
        elif layer.mlp is not None:
            f = layer.mlp
            feed_forward = MixtureFeedForwardSpec(
                hidden_size=cfg.width, n_experts=f.experts, top=f.top, expert_size=f.ff, shared_size=None,
                shared_gate=False, router_bias=True, expert_act="relu2", scoring="softmax_all", n_identity=f.identity,
                groups=f.groups, groups_kept=f.groups_kept, route_scale=f.scale)
        layers.append(LayerSpec(
            mixer=mixer, feed_forward=feed_forward, mixer_norm=norm,
            feed_forward_norm=norm if feed_forward is not None else None, arrangement="pre_norm",
            input_conv=TokenShiftSpec(dim=cfg.width), sublayer_scale=True, depth_mix=(index + 1, total)))
        schedule.append(ScheduleEntry(layer=index, cache=m.kv_from))
    return ModelSpec(
        vocab_size=cfg.vocab, hidden_size=cfg.width, layers=tuple(layers), schedule=tuple(schedule), final_norm=norm,
        tie_word_embeddings=False, max_positions=0, embedding_scale=cfg.embedding_scale,
        stream_parts=(SinusoidPositionSpec(dim=cfg.width, base=POSITION_BASE),))


def weight_targets(cfg: GimudraConfig) -> Dict[str, WeightTarget]:
    width = cfg.width
    vector = dict(role="vector")
    targets: Dict[str, WeightTarget] = {
        "embed": WeightTarget("embed", (cfg.vocab, width)),
        "head": WeightTarget("lm_head", (cfg.vocab, width)),
        "final.norm": WeightTarget("final_norm.weight", (width,), init="ones_jitter", **vector),
    }
    for index, layer in enumerate(cfg.layers):
        m = layer.mixer
        src, dst = f"l{index}", f"layers.{index}"
        targets[f"{src}.norm1"] = WeightTarget(f"{dst}.mixer_norm.weight", (width,), init="ones_jitter", **vector)
        targets[f"{src}.shift"] = WeightTarget(f"{dst}.input_conv.weight", (width,), init="positive", **vector)
        targets[f"{src}.ls1"] = WeightTarget(f"{dst}.mixer_scale", (width,), init="ones_jitter", **vector)
        targets[f"{src}.dwa"] = WeightTarget(f"{dst}.depth_coeff", (index + 2,), init="ones_jitter", **vector)
        q, k, v = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
        targets[f"{src}.mix.q"] = WeightTarget(f"{dst}.mixer.qkv", (q, width), 0)
        targets[f"{src}.mix.q.b"] = WeightTarget(f"{dst}.mixer.qkv_bias", (q,), 0, **vector)
        if m.kv_from is None:
            targets[f"{src}.mix.k"] = WeightTarget(f"{dst}.mixer.qkv", (k, width), q)
            targets[f"{src}.mix.v"] = WeightTarget(f"{dst}.mixer.qkv", (v, width), q + k)
            targets[f"{src}.mix.k.b"] = WeightTarget(f"{dst}.mixer.qkv_bias", (k,), q, **vector)
            targets[f"{src}.mix.v.b"] = WeightTarget(f"{dst}.mixer.qkv_bias", (v,), q + k, **vector)
        # the factor and the slope of the bias by distance: two halves of one vector
        targets[f"{src}.mix.r1"] = WeightTarget(f"{dst}.mixer.log_bias", (m.heads,), 0, init="positive", **vector)
        targets[f"{src}.mix.r2"] = WeightTarget(f"{dst}.mixer.log_bias", (m.heads,), m.heads, init="positive", **vector)
        targets[f"{src}.mix.o"] = WeightTarget(f"{dst}.mixer.out", (width, m.heads * m.vdim))
        if layer.mlp is None:
            continue
        targets[f"{src}.norm2"] = WeightTarget(f"{dst}.feed_forward_norm.weight", (width,), init="ones_jitter", **vector)
        targets[f"{src}.ls2"] = WeightTarget(f"{dst}.feed_forward_scale", (width,), init="ones_jitter", **vector)
        ffn = f"{dst}.feed_forward"
        if isinstance(layer.mlp, DenseConfig):
            ff = layer.mlp.ff
            targets[f"{src}.mlp.gate"] = WeightTarget(f"{ffn}.gate_up", (ff, width), 0)
            targets[f"{src}.mlp.up"] = WeightTarget(f"{ffn}.gate_up", (ff, width), ff)
            targets[f"{src}.mlp.gate.b"] = WeightTarget(f"{ffn}.gate_up_bias", (ff,), 0, **vector)
            targets[f"{src}.mlp.up.b"] = WeightTarget(f"{ffn}.gate_up_bias", (ff,), ff, **vector)
            targets[f"{src}.mlp.down"] = WeightTarget(f"{ffn}.down", (width, ff))
            targets[f"{src}.mlp.down.b"] = WeightTarget(f"{ffn}.down_bias", (width,), **vector)
        else:
            f = layer.mlp
            targets[f"{src}.mlp.router"] = WeightTarget(f"{ffn}.router", (f.experts + f.identity, width))
            targets[f"{src}.mlp.correction"] = WeightTarget(f"{ffn}.router_bias", (f.experts + f.identity,), **vector)
            for e in range(f.experts):
                targets[f"{src}.mlp.e{e}.up"] = WeightTarget(f"{ffn}.up", (f.ff, width), e * f.ff)
                targets[f"{src}.mlp.e{e}.down"] = WeightTarget(f"{ffn}.down", (width, f.ff), e * width)
    return targets


GIMUDRA = register_architecture(
    Architecture(
        name=ARCHITECTURE,
        parse_config=parse_config,
        model_spec=model_spec,
        weight_targets=weight_targets,
        config_to_json=config_to_json,
    ),
    replace=True,
)
