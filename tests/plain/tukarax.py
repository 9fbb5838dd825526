"""Tukarax, the plain way: numpy float64, whole sequences, no cache, one function per
mechanism.  It shares nothing with the product: the tests hold the engine to it.

``config`` is the parsed config.json; ``weights`` maps tensor names to float64 arrays.
"""
from __future__ import annotations

import math

import numpy as np


def rms_norm(x: np.ndarray, w, eps: float) -> np.ndarray:
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * w


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def rotary_frequencies(rot: dict) -> tuple:
    """``(frequencies of the dims/2 pairs, what cosine and sine are multiplied by)``; with
    ``scaling`` the slow pairs turn ``factor`` times slower, the fast ones as they are, those
    between by a ramp over the pair's index."""
    dims, base = rot["dims"], rot["base"]
    i = np.arange(dims // 2, dtype=np.float64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if sc is None:
        return f, 1.0

    def where(turns):  # the (fractional) pair that makes `turns` turns over the original length
        return dims * math.log(sc["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(where(sc["fast"])), 0)
    hi = min(math.ceil(where(sc["slow"])), dims - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / sc["factor"] * ramp + f * (1.0 - ramp), 0.1 * math.log(sc["factor"]) + 1.0


def rotate(x: np.ndarray, rot: dict, neighbours: bool) -> np.ndarray:
    """x: [tokens, heads, dim].  The first ``dims`` elements of every head turn by position times
    frequency: pair i is elements (i, i + dims/2), or with ``neighbours`` (2i, 2i + 1)."""
    dims = rot["dims"]
    f, mult = rotary_frequencies(rot)
    angle = np.arange(x.shape[0], dtype=np.float64)[:, None] * f[None, :]
    c, s = (np.cos(angle) * mult)[:, None, :], (np.sin(angle) * mult)[:, None, :]
    out = x.copy()
    if neighbours:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    else:
        u, v = x[..., : dims // 2], x[..., dims // 2: dims]
        out[..., : dims // 2] = u * c - v * s
        out[..., dims // 2: dims] = v * c + u * s
    return out


def visible(n: int, size) -> np.ndarray:
    i, j = np.arange(n)[:, None], np.arange(n)[None, :]
    seen = j <= i
    return seen if size is None else seen & (i // size == j // size)


def softmax_attention(q, k, v, scale, mask, softcap=None, sink=None) -> np.ndarray:
    """q [n, H, dim], k [n, G, dim], v [n, G, vdim] -> [n, H, vdim].  ``sink`` [H]: one more
    term exp(sink) in every denominator, with no value."""
    n, heads, _ = q.shape
    group = heads // k.shape[1]
    out = np.zeros((n, heads, v.shape[2]))
    for h in range(heads):
        g = h // group
        s = (q[:, h] @ k[:, g].T) * scale
        if softcap is not None:
            s = softcap * np.tanh(s / softcap)
        s = np.where(mask, s, -np.inf)
        top = s.max(axis=-1, keepdims=True)
        if sink is not None:
            top = np.maximum(top, sink[h])
        e = np.exp(s - top)
        denom = e.sum(axis=-1, keepdims=True)
        if sink is not None:
            denom = denom + np.exp(sink[h] - top)
        out[:, h] = (e / denom) @ v[:, g]
    return out


def attention_mixer(h, m: dict, w: dict, pre: str, eps: float) -> np.ndarray:
    """The mixer "attention": halves rotated together, capped scores, chunks, a sink, one gate per head."""
    n = h.shape[0]
    H, G, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[pre + "q"].T).reshape(n, H, dim)
    k = (h @ w[pre + "k"].T).reshape(n, G, dim)
    v = (h @ w[pre + "v"].T).reshape(n, G, vdim)
    if m.get("rot") is not None:
        q, k = rotate(q, m["rot"], False), rotate(k, m["rot"], False)
    size = m["mask"]["size"] if m.get("mask") else None
    o = softmax_attention(q, k, v, m["scale"], visible(n, size), m.get("softcap"), w.get(pre + "sink"))
    gate = sigmoid(h @ w[pre + "g"].T)  # [n, H]
    return (o * gate[:, :, None]).reshape(n, H * vdim) @ w[pre + "o"].T


def keyed_attention(h, m: dict, w: dict, pre: str, eps: float) -> np.ndarray:
    """The left half of "parallel": the values are the projected keys, q and k normed head by head,
    neighbours rotated together, every earlier key, a gate per element."""
    n = h.shape[0]
    H, G, dim = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ w[pre + "q"].T).reshape(n, H, dim)
    k = (h @ w[pre + "k"].T).reshape(n, G, dim)
    v = k.copy()
    q, k = rms_norm(q, w[pre + "q.norm"], eps), rms_norm(k, w[pre + "k.norm"], eps)
    if m.get("rot") is not None:
        q, k = rotate(q, m["rot"], True), rotate(k, m["rot"], True)
    o = softmax_attention(q, k, v, m["scale"], visible(n, None))
    gate = sigmoid(h @ w[pre + "g"].T)
    return (o.reshape(n, -1) * gate) @ w[pre + "o"].T


def causal_conv(x: np.ndarray, taps: np.ndarray) -> np.ndarray:
    """x [n, channels], taps [channels, t]: the last column weighs the current token."""
    n, t = x.shape[0], taps.shape[1]
    padded = np.vstack([np.zeros((t - 1, x.shape[1])), x])
    out = np.zeros_like(x)
    for j in range(t):
        out += padded[j: j + n] * taps[:, j]
    return out


def delta_rule(q, k, v, beta, decay) -> np.ndarray:
    """q, k [n, heads, dim], v [n, heads, vdim], beta and decay [n, heads] -> [n, heads, vdim]."""
    n, heads, dim = q.shape
    out = np.zeros_like(v)
    for h in range(heads):
        S = np.zeros((dim, v.shape[2]))
        for t in range(n):
            S = decay[t, h] * S
            u = beta[t, h] * (v[t, h] - S.T @ k[t, h])
            S = S + np.outer(k[t, h], u)
            out[t, h] = S.T @ q[t, h]
    return out


def delta_mixer(h, m: dict, w: dict, pre: str, eps: float) -> np.ndarray:
    """The right half of "parallel": the gated delta rule."""
    n = h.shape[0]
    heads, G, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(h @ w[pre + "q"].T, w[pre + "q.conv"])).reshape(n, G, dim)
    k = silu(causal_conv(h @ w[pre + "k"].T, w[pre + "k.conv"])).reshape(n, G, dim)
    v = silu(causal_conv(h @ w[pre + "v"].T, w[pre + "v.conv"])).reshape(n, heads, vdim)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * dim ** -0.5
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    rep = heads // G
    q, k = np.repeat(q, rep, axis=1), np.repeat(k, rep, axis=1)
    beta = sigmoid(h @ w[pre + "b"].T)
    decay = np.exp(-np.exp(w[pre + "A_log"]) * softplus(h @ w[pre + "a"].T + w[pre + "dt_bias"]))
    o = delta_rule(q, k, v, beta, decay)
    o = rms_norm(o, w[pre + "norm"], eps) * silu(h @ w[pre + "g"].T).reshape(n, heads, vdim)
    return o.reshape(n, heads * vdim) @ w[pre + "o"].T


def parallel_mixer(h, m: dict, w: dict, pre: str, eps: float) -> np.ndarray:
    left = keyed_attention(h, m["left"], w, pre + "left.", eps)
    right = delta_mixer(h, m["right"], w, pre + "right.", eps)
    return m["left_scale"] * left + m["right_scale"] * right


def route(h, router: np.ndarray, top: int):
    """``(chosen experts [n, top], their weights [n, top], margin [n])``: the scores are sigmoids of
    the router's outputs, the weights the chosen scores as they are; the margin is the distance
    between the last router output taken and the first left, as a share of the token's largest
    output (outputs, not scores: where the sigmoid is flat, scores lie closer together than the
    outputs that rounding moves; a share, because rounding moves an output by a share of its size)."""
    z = h @ router.T
    s = sigmoid(z)
    order = np.argsort(-s, axis=-1, kind="stable")
    chosen = order[:, :top]
    weights = np.take_along_axis(s, chosen, axis=-1)
    if s.shape[1] > top:
        margin = (np.take_along_axis(z, order[:, top - 1: top], axis=-1)
                  - np.take_along_axis(z, order[:, top: top + 1], axis=-1))[:, 0]
        margin = margin / np.maximum(np.abs(z).max(axis=-1), 1e-30)
    else:
        margin = np.full(h.shape[0], np.inf)
    return chosen, weights, margin


def mixture(h, f: dict, w: dict, pre: str, margins=None) -> np.ndarray:
    """Every chosen expert runs on the token's input times its weight."""
    chosen, weights, margin = route(h, w[pre + "router"], f["router"]["top"])
    if margins is not None:
        margins.append(margin)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(chosen[t], weights[t]):
            x = a * h[t]
            p = f"{pre}e{e}."
            out[t] += w[p + "down"] @ (silu(w[p + "gate"] @ x) * (w[p + "up"] @ x))
    return out


MIXERS = {"attention": attention_mixer, "parallel": parallel_mixer}


def forward(config: dict, weights: dict, tokens, streams=None, margins=None) -> np.ndarray:
    """Logits [n, vocab] of a whole sequence.  ``streams``: a list that receives the residual
    stream after every layer; ``margins``: one that receives every router's margins."""
    eps = config["norm"]["eps"]
    x = weights["embed"][np.asarray(tokens)]
    for i, layer in enumerate(config["layers"]):
        pre = f"l{i}."
        x = x + MIXERS[layer["type"]](rms_norm(x, weights[pre + "norm1"], eps), layer["mixer"], weights,
                                      pre + "mix.", eps)
        if layer.get("mlp") is not None:
            x = x + mixture(rms_norm(x, weights[pre + "norm2"], eps), layer["mlp"], weights, pre + "mlp.", margins)
        if streams is not None:
            streams.append(x.copy())
    return rms_norm(x, weights["final.norm"], eps) @ weights["head"].T
