"""Tiny Tukarax configurations for the tests, and model folders made from them."""
from __future__ import annotations

import json
from pathlib import Path

import numpy as np


def _rot(base, dims, scaling=None):
    out = {"base": base, "dims": dims}
    if scaling is not None:
        out["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return out


def _attention(heads, kv_heads, dim, vdim, scale, rot=None, size=None, softcap=None):
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if rot is not None:
        out["rot"] = rot
    if size is not None:
        out["mask"] = {"size": size}
    if softcap is not None:
        out["softcap"] = softcap
    return out


def _delta(heads, kv_heads, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def _parallel(left, right, left_scale, right_scale):
    return {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale}


def _moe(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def _layer(kind, mixer, mlp):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


# A: heads whose sizes are no multiples of 8 (the general kernels everywhere), tiny chunks (every
# prompt crosses many edges), a convolution of two taps, two of five experts a token, a layer
# without feed-forward, a capped, stretched and fully rotated attention beside a plain one.
TUKARAX_A = {
    "architecture": "Tukarax", "vocab": 113, "width": 40, "norm": {"eps": 2e-5},
    "layers": [
        _layer("parallel", _parallel(_attention(4, 2, 12, 12, 0.3, _rot(10000.0, 6)), _delta(4, 2, 12, 20, 2), 0.7, 1.6),
               _moe(5, 2, 16)),
        _layer("attention", _attention(4, 2, 12, 20, 0.4, _rot(5000.0, 12, (4.0, 16, 4.0, 1.0)), 7, 3.0), None),
        _layer("attention", _attention(2, 1, 10, 6, 0.5, _rot(300.0, 4), 5), _moe(4, 4, 8)),
        _layer("parallel", _parallel(_attention(3, 3, 10, 10, 0.25), _delta(2, 2, 6, 4, 5), 1.0, 1.0), _moe(3, 1, 24)),
    ],
}
# B: sizes that the matrix-core attention kernels take for the left mixer (heads of 64), attention
# first, chunks that are no multiple of a page or a block of keys, three of six experts with sizes
# the sorted expert path takes, four taps, more value heads than q/k heads in the delta rule.
TUKARAX_B = {
    "architecture": "Tukarax", "vocab": 160, "width": 64, "norm": {"eps": 1e-6},
    "layers": [
        _layer("attention", _attention(6, 2, 64, 64, 0.11, _rot(1.0e6, 32, (8.0, 64, 16.0, 2.0)), 50, 30.0), _moe(6, 3, 40)),
        _layer("parallel", _parallel(_attention(2, 1, 64, 64, 0.12, _rot(5.0e5, 32)), _delta(4, 1, 32, 64, 4), 1.3, 0.4),
               _moe(8, 1, 24)),
        _layer("attention", _attention(3, 3, 32, 48, 0.2, _rot(1.0e4, 16), 128, 10.0), _moe(7, 2, 24)),
    ],
}
# C: heads of 128 on both sides (the delta rule's widest slices), one key/value head for eight
# heads on the left, as many q/k heads as value heads on the right, chunks longer than any prompt,
# every expert taken, scales of one.
TUKARAX_C = {
    "architecture": "Tukarax", "vocab": 97, "width": 128, "norm": {"eps": 3e-6},
    "layers": [
        _layer("parallel", _parallel(_attention(8, 1, 128, 128, 0.09, _rot(2.0e4, 128)), _delta(2, 2, 128, 128, 3), 1.0, 1.0),
               _moe(2, 2, 64)),
        _layer("attention", _attention(4, 4, 16, 24, 0.25, _rot(1.0e4, 8, (2.0, 32, 8.0, 1.0)), 1000, 50.0), _moe(4, 1, 32)),
    ],
}
# D: a delta rule whose heads of 256 are cut over four threads a column, a convolution of one tap
# (no window to keep), values larger than keys in attention, a chunk of one page, a left mixer
# without rotation, a layer without feed-forward first.
TUKARAX_D = {
    "architecture": "Tukarax", "vocab": 203, "width": 96, "norm": {"eps": 1e-5},
    "layers": [
        _layer("parallel", _parallel(_attention(4, 2, 24, 24, 0.2), _delta(2, 1, 256, 64, 1), 0.5, 2.0), None),
        _layer("attention", _attention(4, 2, 40, 72, 0.16, _rot(1.0e4, 40), 64, 20.0), _moe(9, 4, 32)),
        _layer("parallel", _parallel(_attention(2, 2, 128, 128, 0.1, _rot(1.0e5, 64)), _delta(3, 3, 40, 24, 8), 1.1, 0.9),
               _moe(5, 2, 48)),
    ],
}
# E: nothing is a multiple of 8: a width of 100, experts of 20 hidden units, a vocabulary of 301, heads
# of 20, 12 and 10 elements: every product and every expert path falls back to its general kernel.
TUKARAX_E = {
    "architecture": "Tukarax", "vocab": 301, "width": 100, "norm": {"eps": 1e-6},
    "layers": [
        _layer("attention", _attention(5, 5, 12, 10, 0.3, _rot(1.0e4, 6, (3.0, 20, 5.0, 1.0)), 9, 7.0), _moe(3, 2, 20)),
        _layer("parallel", _parallel(_attention(2, 1, 20, 20, 0.2, _rot(777.0, 10)), _delta(4, 2, 10, 6, 3), 0.9, 1.1),
               _moe(11, 5, 12)),
    ],
}
CONFIGS = {"A": TUKARAX_A, "B": TUKARAX_B, "C": TUKARAX_C, "D": TUKARAX_D, "E": TUKARAX_E}


def make_folder(tmp: Path, name: str, *, dtype: str = "float32", seed: int = 5, std: float = 0.12,
                router_scale: float = 6.0, config=None) -> Path:
    """A model folder of random weights changed after drawing so that faults show: routers scaled up
    (clear choices: the tests do not rest on close calls), sinks as large as scores, decays close
    to one (a lost state is missed for many tokens), convolutions that weigh every tap, norm
    weights that differ from one."""
    from safetensors.torch import load_file, save_file

    from pylon_amd.weights import write_random_model

    folder = write_random_model(Path(tmp) / f"tukarax_{name}_{dtype}_{seed}", config or CONFIGS[name], seed,
                                dtype=dtype, std=std, norm_jitter=0.2)
    path = folder / "model.safetensors"
    tensors = load_file(str(path))
    for key in list(tensors):
        value = tensors[key].float()
        if key.endswith(".mlp.router"):
            value = value * router_scale
        elif key.endswith(".sink"):
            value = value * 12.0
        elif key.endswith(".A_log"):
            value = value * 6.0 - 2.5
        elif key.endswith(".conv"):
            value = value * 5.0
        elif key.endswith(".right.b") or key.endswith(".right.a"):
            value = value * 4.0
        else:
            continue
        tensors[key] = value.to(tensors[key].dtype)
    save_file(tensors, str(path))
    return folder


def read_folder(folder: Path):
    import torch
    from safetensors.torch import load_file

    cfg = json.loads((Path(folder) / "config.json").read_text())
    weights = {name: t.to(torch.float64).numpy() for name, t in load_file(str(Path(folder) / "model.safetensors")).items()}
    return cfg, weights


def tokens(vocab: int, count: int, seed: int):
    return np.random.default_rng(seed).integers(0, vocab, count).tolist()
