"""Gimudra, the plain way: numpy float64, whole sequences, no cache, one function per
mechanism.  It shares nothing with the product: the tests hold the engine to it.

``config`` is the parsed config.json; ``weights`` maps tensor names to float64 arrays.
"""
from __future__ import annotations

import numpy as np


def rms_norm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * w


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def sinusoid(n: int, width: int, base: float = 10000.0) -> np.ndarray:
    """Position vectors of positions 0 .. n - 1: element 2i the sine, 2i + 1 the cosine of
    ``p * base ** (-2i / width)``."""
    out = np.zeros((n, width))
    p = np.arange(n, dtype=np.float64)[:, None]
    for e in range(width):
        i = e // 2
        angle = p[:, 0] * base ** (-2.0 * i / width)
        out[:, e] = np.sin(angle) if e % 2 == 0 else np.cos(angle)
    return out


def embed(tokens, table: np.ndarray, scale: float) -> np.ndarray:
    x = table[np.asarray(tokens)] * scale
    return x + sinusoid(len(tokens), table.shape[1])


def token_shift(h: np.ndarray, shift: np.ndarray) -> np.ndarray:
    """Every token's input moved towards the previous token's (zeros before the first)."""
    before = np.vstack([np.zeros((1, h.shape[1])), h[:-1]])
    return h + (before - h) * shift


def chunk_mask(n: int, size) -> np.ndarray:
    i, j = np.arange(n)[:, None], np.arange(n)[None, :]
    seen = j <= i
    return seen if size is None else seen & (i // size == j // size)


def distance_bias(r1: np.ndarray, r2: np.ndarray, n: int) -> np.ndarray:
    """[heads, n, n]: what is taken off the score of query i and key j (0 where j > i)."""
    far = np.maximum(np.arange(n)[:, None] - np.arange(n)[None, :], 0).astype(np.float64)
    return r1[:, None, None] * np.log(1.0 + r2[:, None, None] * far[None])


def softmax_masked(scores: np.ndarray, visible: np.ndarray) -> np.ndarray:
    s = np.where(visible, scores, -np.inf)
    s = s - s.max(axis=-1, keepdims=True)
    e = np.where(visible, np.exp(s), 0.0)
    return e / e.sum(axis=-1, keepdims=True)


def project(h, weights, name):
    return h @ weights[name].T + weights[name + ".b"]


def keys_and_values(h, weights, prefix, m):
    n = h.shape[0]
    k = project(h, weights, prefix + "k").reshape(n, m["kv_heads"], m["dim"])
    v = project(h, weights, prefix + "v").reshape(n, m["kv_heads"], m["vdim"])
    return k, v


def attention(h, weights, prefix, m, kv):
    """``kv``: the keys and values this layer attends over (its own, or an earlier layer's)."""
    n = h.shape[0]
    heads, groups = m["heads"], m["kv_heads"]
    q = project(h, weights, prefix + "q").reshape(n, heads, m["dim"])
    k, v = kv
    visible = chunk_mask(n, (m.get("mask") or {}).get("size"))
    bias = distance_bias(weights[prefix + "r1"], weights[prefix + "r2"], n)
    out = np.zeros((n, heads, m["vdim"]))
    for head in range(heads):
        g = head // (heads // groups)
        scores = (q[:, head] @ k[:, g].T) * m["scale"] - bias[head]
        out[:, head] = softmax_masked(scores, visible) @ v[:, g]
    return out.reshape(n, heads * m["vdim"]) @ weights[prefix + "o"].T


def dense(h, weights, prefix):
    hidden = silu(project(h, weights, prefix + "gate")) * project(h, weights, prefix + "up")
    return project(hidden, weights, prefix + "down")


def route(h, weights, prefix, router):
    """Per token: the chosen router outputs, their weights, and how clear the choice was (the
    smallest gap, in corrected scores, between something taken and something left)."""
    experts, identity, top = router["experts"], router.get("identity", 0), router["top"]
    outputs = experts + identity
    groups = router.get("groups") or {"count": 1, "keep": 1}
    count, keep = groups["count"], groups["keep"]
    z = h @ weights[prefix + "router"].T
    z = z - z.max(axis=-1, keepdims=True)
    scores = np.exp(z) / np.exp(z).sum(axis=-1, keepdims=True)
    chosen, chosen_w, margin = [], [], []
    for t in range(h.shape[0]):
        choice = scores[t] + weights[prefix + "correction"]
        best = choice.reshape(count, outputs // count).max(axis=1)
        order = sorted(range(count), key=lambda g: (-best[g], g))
        kept, gap = set(order[:keep]), np.inf
        if keep < count:
            gap = best[order[keep - 1]] - best[order[keep]]
        allowed = [e for e in range(outputs) if e // (outputs // count) in kept]
        ranked = sorted(allowed, key=lambda e: (-choice[e], e))
        if top < len(ranked):
            gap = min(gap, choice[ranked[top - 1]] - choice[ranked[top]])
        chosen.append(ranked[:top])
        chosen_w.append([scores[t, e] * router.get("scale", 1.0) for e in ranked[:top]])
        margin.append(gap)
    return chosen, chosen_w, np.asarray(margin)


def mixture(h, weights, prefix, mlp, margins=None):
    router = mlp["router"]
    chosen, chosen_w, margin = route(h, weights, prefix, router)
    if margins is not None:
        margins.append(margin)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(chosen[t], chosen_w[t]):
            if e >= router["experts"]:
                out[t] += w * h[t]  # an identity expert
            else:
                hidden = np.maximum(weights[f"{prefix}e{e}.up"] @ h[t], 0.0) ** 2
                out[t] += w * (weights[f"{prefix}e{e}.down"] @ hidden)
    return out


def depth_mix(streams, coeff) -> np.ndarray:
    return sum(c * s for c, s in zip(coeff, streams))


def forward(config, weights, tokens, margins=None, keep_layers=False):
    """Logits [tokens, vocab]; with ``keep_layers`` also the stream after every layer (mixed)."""
    eps = config["norm"]["eps"]
    x = embed(tokens, weights["embed"], (config.get("embedding") or {}).get("scale", 1.0))
    streams, kept, cached = [x], [], {}
    for index, layer in enumerate(config["layers"]):
        p = f"l{index}."
        m = layer["mixer"]
        h = token_shift(rms_norm(x, weights[p + "norm1"], eps), weights[p + "shift"])
        if m.get("kv_from") is None:
            cached[index] = keys_and_values(h, weights, p + "mix.", m)
        x = x + attention(h, weights, p + "mix.", m, cached[m.get("kv_from", index) if m.get("kv_from") is not None else index]) * weights[p + "ls1"]
        if layer.get("mlp") is not None:
            h = rms_norm(x, weights[p + "norm2"], eps)
            if layer["mlp"]["kind"] == "dense":
                f = dense(h, weights, p + "mlp.")
            else:
                f = mixture(h, weights, p + "mlp.", layer["mlp"], margins)
            x = x + f * weights[p + "ls2"]
        streams.append(x)
        x = depth_mix(streams, weights[p + "dwa"])
        kept.append(x)
    logits = rms_norm(x, weights["final.norm"], eps) @ weights["head"].T
    return (logits, kept) if keep_layers else logits
