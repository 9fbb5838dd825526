"""Tiny Gimudra configurations for the tests, and model folders made from them."""
from __future__ import annotations

import json
from pathlib import Path

import numpy as np


def _attention(heads, kv_heads, dim, vdim, scale, size=None, kv_from=None):
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if size is not None:
        out["mask"] = {"size": size}
    if kv_from is not None:
        out["kv_from"] = kv_from
    return out


def _moe(experts, identity, top, ff, count, keep, scale):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "identity": identity, "top": top, "scale": scale,
                       "groups": {"count": count, "keep": keep}}}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _layer(mixer, mlp):
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


# P: heads whose sizes are no multiples of 8 (the general attention kernel), tiny chunks (every prompt
# crosses many edges), a dense feed-forward first, layers on an earlier layer's keys and values (one of
# them with chunks of another size: that cache keeps every token), a layer without feed-forward, a
# mixture without identity experts and without groups in which a token takes every expert.
GIMUDRA_P = {
    "architecture": "Gimudra", "vocab": 113, "width": 40, "norm": {"eps": 2e-5}, "embedding": {"scale": 1.7},
    "layers": [
        _layer(_attention(4, 2, 12, 20, 0.3, 7), _dense(24)),
        _layer(_attention(4, 2, 12, 20, 0.4, 7, kv_from=0), _moe(5, 1, 2, 16, 3, 2, 1.5)),
        _layer(_attention(2, 1, 10, 6, 0.5, 5), None),
        _layer(_attention(4, 2, 12, 20, 0.2, 9, kv_from=0), _moe(4, 0, 4, 8, 1, 1, 1.0)),
    ],
}
# Q: head sizes that the matrix-core kernel takes, chunks that are no multiple of a block of keys and
# chunks of several blocks, a mixture first, a dense feed-forward later, one key/value head per head,
# an embedding scale of one.
GIMUDRA_Q = {
    "architecture": "Gimudra", "vocab": 160, "width": 64, "norm": {"eps": 1e-6}, "embedding": {"scale": 1.0},
    "layers": [
        _layer(_attention(6, 2, 32, 24, 0.18, 50), _moe(6, 2, 3, 40, 4, 2, 0.7)),
        _layer(_attention(6, 2, 32, 24, 0.25, 50, kv_from=0), _dense(72)),
        _layer(_attention(3, 3, 64, 64, 0.125, 128), _moe(7, 1, 2, 24, 2, 1, 2.5)),
        _layer(_attention(3, 3, 64, 64, 0.1, 128, kv_from=2), None),
    ],
}
# R: one key/value head for all heads, a layer without any mask (every earlier key: the bias by
# distance is then evaluated in the kernel), chunks longer than any prompt, more identity experts
# than experts and more of them taken by a token than there are experts, groups of one output each,
# all of them kept.
GIMUDRA_R = {
    "architecture": "Gimudra", "vocab": 97, "width": 48, "norm": {"eps": 3e-6}, "embedding": {"scale": 0.25},
    "layers": [
        _layer(_attention(5, 1, 16, 8, 0.25), _dense(20)),
        _layer(_attention(2, 2, 8, 12, 0.35, 1000), _moe(2, 3, 3, 12, 5, 5, 3.0)),
    ],
}
# S: sizes for the matrix-core kernels over pages of 64, sixteen query heads on one key/value head
# (a whole tile of columns in a step of single tokens), eight experts with sizes that the sorted
# expert path takes.
GIMUDRA_S = {
    "architecture": "Gimudra", "vocab": 203, "width": 128, "norm": {"eps": 1e-5}, "embedding": {"scale": 2.0},
    "layers": [
        _layer(_attention(16, 1, 16, 8, 0.25, 96), _moe(8, 0, 2, 64, 4, 3, 1.0)),
        _layer(_attention(4, 4, 40, 36, 0.16, 33), _moe(6, 6, 4, 32, 6, 4, 1.25)),
        _layer(_attention(4, 4, 40, 36, 0.2, 33, kv_from=1), _dense(96)),
    ],
}
CONFIGS = {"P": GIMUDRA_P, "Q": GIMUDRA_Q, "R": GIMUDRA_R, "S": GIMUDRA_S}


def make_folder(tmp: Path, name: str, *, dtype: str = "float32", seed: int = 5, std: float = 0.12,
                router_scale: float = 6.0, config=None) -> Path:
    """A model folder of random weights in which routers are scaled up after drawing (clear choices:
    the tests do not rest on close calls), the corrections are as large as the scores they correct,
    and norm weights, layer scales and mixing coefficients differ from one."""
    from safetensors.torch import load_file, save_file

    from pylon_amd.weights import write_random_model

    folder = write_random_model(Path(tmp) / f"gimudra_{name}_{dtype}_{seed}", config or CONFIGS[name], seed,
                                dtype=dtype, std=std, norm_jitter=0.2)
    path = folder / "model.safetensors"
    tensors = load_file(str(path))
    for key in list(tensors):
        if key.endswith(".mlp.router"):
            tensors[key] = (tensors[key].float() * router_scale).to(tensors[key].dtype)
        if key.endswith(".dwa"):  # a mix, not a sum: the streams stay of one size through the layers
            tensors[key] = (tensors[key].float() / tensors[key].numel() ** 0.5).to(tensors[key].dtype)
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
