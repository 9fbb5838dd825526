"""Tukarax: config.json keys, the model as specs, and checkpoint tensor names.

A decoder whose layers are listed one by one in ``layers``; each entry has a ``type`` (the mixer:
"attention" or "parallel"), the mixer's sizes under ``mixer`` and its feed-forward under ``mlp``
(null: none).  A layer is pre-normed (RMS norms with ``norm.eps``).

* "attention": grouped queries with keys of ``dim`` and values of ``vdim`` elements; the first
  ``rot.dims`` elements of every head of q and k turn by the position, element ``i`` together with
  ``i + dims/2``, with frequencies ``rot.base ** (-2i/dims)`` that ``rot.scaling`` (factor, original,
  fast, slow) stretches for long contexts; ``scale`` from the config; scores capped by ``softcap *
  tanh(s / softcap)``; position ``i`` sees key ``j <= i`` only inside its own chunk of ``mask.size``
  positions; a learned sink per head in the softmax's denominator; every head's output times
  ``sigmoid(W_g h)`` of that head.
* "parallel": ``left_scale * left(h) + right_scale * right(h)``.  Left: attention whose values are the
  keys as projected (no value projection), q and k normed head by head with one weight for all heads,
  neighbours ``(2i, 2i + 1)`` turned together, every earlier key visible, plain softmax, the
  concatenated heads times ``sigmoid(W_g h)`` element by element.  Right: the gated delta rule
  (:class:`~pylon_amd.config.specs.DeltaRuleSpec`) with ``conv`` taps.
* Feed-forward "moe": ``experts`` gated experts of ``expert.ff`` hidden units; the scores are the
  sigmoids of the router's outputs, a token takes the ``top`` largest, and each chosen expert runs on
  the token's input times its score.
* The final norm, then the head (a matrix of its own).

Keys that a mixer's entry leaves out switch the mechanism off: no ``rot``, no rotation; no
``rot.scaling``, plain frequencies; no ``softcap``, no cap; no ``mask``, every earlier key.

Tensors: ``embed``, ``head``, ``final.norm``, per layer ``l<i>.norm1``, ``.norm2``; attention
``.mix.{q,k,v,g,o}``, ``.mix.sink``; parallel ``.mix.left.{q,k,g,o}``, ``.mix.left.{q,k}.norm``,
``.mix.right.{q,k,v,g,b,a,o}``, ``.mix.right.{q,k,v}.conv``, ``.mix.right.{A_log,dt_bias,norm}``;
mixture ``.mlp.e<j>.{gate,up,down}``, ``.mlp.router``.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, Mapping, Optional, Tuple

from ..config.registry import Architecture, WeightTarget, register_architecture
from ..config.specs import (
    AttentionSpec,
    DeltaRuleSpec,
    LayerSpec,
    MixtureFeedForwardSpec,
    ModelSpec,
    NormSpec,
    ParallelMixerSpec,
    PositionSpec,
    RotaryScalingSpec,
    ScheduleEntry,
)

ARCHITECTURE = "Tukarax"

UNIT_EPS = 1e-6  # inside the root that makes the delta rule's q and k unit vectors


def _positive_int(value, name: str) -> int:
    if isinstance(value, bool) or not isinstance(value, int) or value < 1:
        raise ValueError(f"{name} must be a positive integer, got {value!r}")
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
class RotaryConfig:
    base: float
    dims: int
    scaling: Optional[Tuple[float, float, float, float]]  # factor, original, fast, slow


@dataclass(frozen=True)
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[RotaryConfig]
    softcap: Optional[float] = None
    mask_size: Optional[int] = None


@dataclass(frozen=True)
class DeltaConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int


@dataclass(frozen=True)
class ParallelConfig:
    left: AttentionConfig
    right: DeltaConfig
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class MixtureConfig:
    experts: int
    top: int
    ff: int


@dataclass(frozen=True)
class LayerConfig:
    type: str
    mixer: object  # AttentionConfig or ParallelConfig
    mlp: Optional[MixtureConfig]


@dataclass(frozen=True)
class TukaraxConfig:
    vocab: int
    width: int
    layers: Tuple[LayerConfig, ...]
    norm_eps: float
    initializer_range: float = 0.02  # only used to draw random weights
    eos_token_id: Optional[Tuple[int, ...]] = None


def _parse_rot(rot: Optional[Mapping], dim: int, where: str) -> Optional[RotaryConfig]:
    if rot is None:
        return None
    _require(rot, ("base", "dims"), where)
    dims = _positive_int(rot["dims"], "rot.dims")
    if dims % 2 or dims > dim:
        raise ValueError(f"{where}: rot.dims {dims} must be even and at most the head's {dim} elements")
    scaling = rot.get("scaling")
    if scaling is not None:
        _require(scaling, ("factor", "original", "fast", "slow"), where + ".scaling")
        scaling = tuple(_positive(scaling[key], f"rot.scaling.{key}") for key in ("factor", "original", "fast", "slow"))
    return RotaryConfig(_positive(rot["base"], "rot.base"), dims, scaling)


def _parse_attention(m: Mapping, where: str) -> AttentionConfig:
    _require(m, ("heads", "kv_heads", "dim", "vdim", "scale"), where)
    heads, kv_heads = _positive_int(m["heads"], "heads"), _positive_int(m["kv_heads"], "kv_heads")
    if heads % kv_heads:
        raise ValueError("The number of Q heads must be divisible by the number of KV heads.")
    dim = _positive_int(m["dim"], "dim")
    mask = m.get("mask")
    size = None
    if mask is not None:
        _require(mask, ("size",), where + ".mask")
        size = _positive_int(mask["size"], "mask.size")
    softcap = m.get("softcap")
    return AttentionConfig(heads, kv_heads, dim, _positive_int(m["vdim"], "vdim"), _positive(m["scale"], "scale"),
                           _parse_rot(m.get("rot"), dim, where + ".rot"),
                           None if softcap is None else _positive(softcap, "softcap"), size)


def _parse_mixer(kind: str, m: Mapping, where: str):
    if kind == "attention":
        return _parse_attention(m, where)
    if kind != "parallel":
        raise ValueError(f"{where}: unknown layer type {kind!r} (known: attention, parallel)")
    _require(m, ("left", "right", "left_scale", "right_scale"), where)
    left = _parse_attention(m["left"], where + ".left")
    if left.vdim != left.dim:
        raise ValueError(f"{where}.left: the values are the keys, so vdim {left.vdim} must equal dim {left.dim}")
    if left.softcap is not None or left.mask_size is not None:
        raise ValueError(f"{where}.left: the left mixer sees every earlier key and caps no score")
    r = m["right"]
    _require(r, ("heads", "kv_heads", "dim", "vdim", "conv"), where + ".right")
    heads, kv_heads = _positive_int(r["heads"], "heads"), _positive_int(r["kv_heads"], "kv_heads")
    if heads % kv_heads:
        raise ValueError("The number of value heads must be divisible by the number of q/k heads.")
    right = DeltaConfig(heads, kv_heads, _positive_int(r["dim"], "dim"), _positive_int(r["vdim"], "vdim"),
                        _positive_int(r["conv"], "conv"))
    return ParallelConfig(left, right, float(m["left_scale"]), float(m["right_scale"]))


def _parse_mlp(mlp: Optional[Mapping], where: str) -> Optional[MixtureConfig]:
    if mlp is None:
        return None
    _require(mlp, ("kind",), where)
    if mlp["kind"] != "moe":
        raise ValueError(f"{where}: unknown feed-forward kind {mlp['kind']!r} (known: moe)")
    _require(mlp, ("expert", "router"), where)
    _require(mlp["expert"], ("ff",), where + ".expert")
    _require(mlp["router"], ("experts", "top"), where + ".router")
    experts, top = _positive_int(mlp["router"]["experts"], "experts"), _positive_int(mlp["router"]["top"], "top")
    if top > experts:
        raise ValueError(f"{where}: top {top} exceeds the {experts} experts")
    return MixtureConfig(experts, top, _positive_int(mlp["expert"]["ff"], "expert.ff"))


def parse_config(data: Mapping) -> TukaraxConfig:
    _require(data, ("vocab", "width", "layers", "norm"), "the model")
    _require(data["norm"], ("eps",), "norm")
    layers = []
    for index, entry in enumerate(data["layers"]):
        where = f"layers[{index}]"
        _require(entry, ("type", "mixer"), where)
        layers.append(LayerConfig(entry["type"], _parse_mixer(entry["type"], entry["mixer"], where + ".mixer"),
                                  _parse_mlp(entry.get("mlp"), where + ".mlp")))
    if not layers:
        raise ValueError("the model has no layers")
    eos = data.get("eos_token_id")
    if isinstance(eos, int):
        eos = (eos,)
    elif eos is not None:
        eos = tuple(int(v) for v in eos)
    return TukaraxConfig(
        vocab=_positive_int(data["vocab"], "vocab"), width=_positive_int(data["width"], "width"),
        layers=tuple(layers), norm_eps=_positive(data["norm"]["eps"], "norm.eps"),
        initializer_range=float(data.get("initializer_range", 0.02)), eos_token_id=eos)


def _attention_json(m: AttentionConfig) -> dict:
    out = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale}
    if m.rot is not None:
        out["rot"] = {"base": m.rot.base, "dims": m.rot.dims}
        if m.rot.scaling is not None:
            out["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), m.rot.scaling))
    if m.softcap is not None:
        out["softcap"] = m.softcap
    if m.mask_size is not None:
        out["mask"] = {"size": m.mask_size}
    return out


def config_to_json(cfg: TukaraxConfig) -> dict:
    layers = []
    for layer in cfg.layers:
        m = layer.mixer
        if isinstance(m, ParallelConfig):
            r = m.right
            mixer = {"left": _attention_json(m.left), "left_scale": m.left_scale,
                     "right": {"heads": r.heads, "kv_heads": r.kv_heads, "dim": r.dim, "vdim": r.vdim, "conv": r.conv},
                     "right_scale": m.right_scale}
        else:
            mixer = _attention_json(m)
        mlp = None
        if layer.mlp is not None:
            f = layer.mlp
            mlp = {"kind": "moe", "expert": {"ff": f.ff}, "router": {"experts": f.experts, "top": f.top}}
        layers.append({"type": layer.type, "mixer": mixer, "mlp": mlp})
    out = {"architecture": ARCHITECTURE, "vocab": cfg.vocab, "width": cfg.width, "layers": layers,
           "norm": {"eps": cfg.norm_eps}, "initializer_range": cfg.initializer_range}
    if cfg.eos_token_id is not None:
        out["eos_token_id"] = list(cfg.eos_token_id)
    return out


def _position(rot: Optional[RotaryConfig], neighbours: bool) -> PositionSpec:
    if rot is None:
        return PositionSpec(kind="none")
    scaling = None if rot.scaling is None else RotaryScalingSpec(*rot.scaling)
    return PositionSpec(kind="rope", theta=rot.base, rotary_dim=rot.dims, interleaved=neighbours, scaling=scaling)


def _mixer_spec(cfg: TukaraxConfig, layer: LayerConfig):
    m = layer.mixer
    if isinstance(m, AttentionConfig):
        return AttentionSpec(
            hidden_size=cfg.width, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim, scale=m.scale,
            position=_position(m.rot, False), qk_norm=False, v_head_dim=m.vdim, chunk=m.mask_size, softcap=m.softcap,
            sink=True, output_gate="head")
    left = AttentionSpec(
        hidden_size=cfg.width, n_heads=m.left.heads, n_kv_heads=m.left.kv_heads, head_dim=m.left.dim,
        scale=m.left.scale, position=_position(m.left.rot, True), qk_norm=True, qk_norm_eps=cfg.norm_eps,
        qk_norm_over="head", v_head_dim=m.left.vdim, output_gate="element", values_from_keys=True)
    right = DeltaRuleSpec(
        hidden_size=cfg.width, n_heads=m.right.heads, n_kv_heads=m.right.kv_heads, head_dim=m.right.dim,
        v_head_dim=m.right.vdim, conv_taps=m.right.conv, norm_eps=cfg.norm_eps, unit_eps=UNIT_EPS)
    return ParallelMixerSpec(left=left, right=right, left_scale=m.left_scale, right_scale=m.right_scale)


def model_spec(cfg: TukaraxConfig) -> ModelSpec:
    norm = NormSpec(kind="rmsnorm", dim=cfg.width, eps=cfg.norm_eps)
    layers, schedule = [], []
    for index, layer in enumerate(cfg.layers):
        feed_forward = None
        if layer.mlp is not None:
            f = layer.mlp
            feed_forward = MixtureFeedForwardSpec(
                hidden_size=cfg.width, n_experts=f.experts, top=f.top, expert_size=f.ff, shared_size=None,
                shared_gate=False, router_bias=False, scoring="sigmoid", weight_on_input=True)
        layers.append(LayerSpec(
            mixer=_mixer_spec(cfg, layer), feed_forward=feed_forward, mixer_norm=norm,
            feed_forward_norm=norm if feed_forward is not None else None, arrangement="pre_norm"))
        schedule.append(ScheduleEntry(layer=index))
    return ModelSpec(
        vocab_size=cfg.vocab, hidden_size=cfg.width, layers=tuple(layers), schedule=tuple(schedule), final_norm=norm,
        tie_word_embeddings=False, max_positions=0)


def _attention_targets(targets: Dict[str, WeightTarget], src: str, dst: str, m: AttentionConfig, width: int,
                       *, keyed: bool) -> None:
    """``keyed``: the left mixer of a parallel layer (no value projection, head norms, a gate per element)."""
    vector = dict(role="vector")
    q, k = m.heads * m.dim, m.kv_heads * m.dim
    v = 0 if keyed else m.kv_heads * m.vdim
    targets[f"{src}.q"] = WeightTarget(f"{dst}.qkv", (q, width), 0)
    targets[f"{src}.k"] = WeightTarget(f"{dst}.qkv", (k, width), q)
    if keyed:
        targets[f"{src}.q.norm"] = WeightTarget(f"{dst}.q_norm", (m.dim,), init="ones_jitter", **vector)
        targets[f"{src}.k.norm"] = WeightTarget(f"{dst}.k_norm", (m.dim,), init="ones_jitter", **vector)
        targets[f"{src}.g"] = WeightTarget(f"{dst}.qkv", (m.heads * m.vdim, width), q + k)
    else:
        targets[f"{src}.v"] = WeightTarget(f"{dst}.qkv", (v, width), q + k)
        targets[f"{src}.g"] = WeightTarget(f"{dst}.qkv", (m.heads, width), q + k + v)
        targets[f"{src}.sink"] = WeightTarget(f"{dst}.sink", (m.heads,), **vector)
    targets[f"{src}.o"] = WeightTarget(f"{dst}.out", (width, m.heads * m.vdim))


def _delta_targets(targets: Dict[str, WeightTarget], src: str, dst: str, r: DeltaConfig, width: int) -> None:
    vector = dict(role="vector")
    qk, v = r.kv_heads * r.dim, r.heads * r.vdim
    rows = {"q": (qk, 0), "k": (qk, qk), "v": (v, 2 * qk), "g": (v, 2 * qk + v), "b": (r.heads, 2 * qk + 2 * v),
            "a": (r.heads, 2 * qk + 2 * v + r.heads)}
    for name, (count, start) in rows.items():
        targets[f"{src}.{name}"] = WeightTarget(f"{dst}.proj", (count, width), start)
    for name in ("q", "k", "v"):
        count, start = rows[name]
        targets[f"{src}.{name}.conv"] = WeightTarget(f"{dst}.conv", (count, r.conv), start, **vector)
    targets[f"{src}.A_log"] = WeightTarget(f"{dst}.a_log", (r.heads,), **vector)
    targets[f"{src}.dt_bias"] = WeightTarget(f"{dst}.dt_bias", (r.heads,), **vector)
    targets[f"{src}.norm"] = WeightTarget(f"{dst}.norm", (r.vdim,), init="ones_jitter", **vector)
    targets[f"{src}.o"] = WeightTarget(f"{dst}.out", (width, v))


def weight_targets(cfg: TukaraxConfig) -> Dict[str, WeightTarget]:
    width = cfg.width
    vector = dict(role="vector")
    targets: Dict[str, WeightTarget] = {
        "embed": WeightTarget("embed", (cfg.vocab, width)),
        "head": WeightTarget("lm_head", (cfg.vocab, width)),
        "final.norm": WeightTarget("final_norm.weight", (width,), init="ones_jitter", **vector),
    }
    for index, layer in enumerate(cfg.layers):
        src, dst = f"l{index}", f"layers.{index}"
        targets[f"{src}.norm1"] = WeightTarget(f"{dst}.mixer_norm.weight", (width,), init="ones_jitter", **vector)
        if isinstance(layer.mixer, ParallelConfig):
            _attention_targets(targets, f"{src}.mix.left", f"{dst}.mixer.left", layer.mixer.left, width, keyed=True)
            _delta_targets(targets, f"{src}.mix.right", f"{dst}.mixer.right", layer.mixer.right, width)
        else:
            _attention_targets(targets, f"{src}.mix", f"{dst}.mixer", layer.mixer, width, keyed=False)
        if layer.mlp is None:
            continue
        f = layer.mlp
        ffn = f"{dst}.feed_forward"
        targets[f"{src}.norm2"] = WeightTarget(f"{dst}.feed_forward_norm.weight", (width,), init="ones_jitter", **vector)
        targets[f"{src}.mlp.router"] = WeightTarget(f"{ffn}.router", (f.experts, width))
        for e in range(f.experts):
            targets[f"{src}.mlp.e{e}.gate"] = WeightTarget(f"{ffn}.gate_up", (f.ff, width), e * 2 * f.ff)
            targets[f"{src}.mlp.e{e}.up"] = WeightTarget(f"{ffn}.gate_up", (f.ff, width), e * 2 * f.ff + f.ff)
            targets[f"{src}.mlp.e{e}.down"] = WeightTarget(f"{ffn}.down", (width, f.ff), e * width)
    return targets


TUKARAX = register_architecture(
    Architecture(
        name=ARCHITECTURE,
        parse_config=parse_config,
        model_spec=model_spec,
        weight_targets=weight_targets,
        config_to_json=config_to_json,
    ),
    replace=True,
)
