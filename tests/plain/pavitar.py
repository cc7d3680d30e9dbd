"""Pavitar, the plain way: numpy float64, whole sequences, no cache, one function per
mechanism.  It shares nothing with the product: the tests hold the engine to it.

``config`` is the parsed config.json; ``weights`` maps tensor names to float64 arrays.
"""
from __future__ import annotations

import numpy as np


def unit_rms(x: np.ndarray, eps: float) -> np.ndarray:
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def norm_around_zero(x, w, eps):
    """The layer norm of the design: the stored weight is the distance from one."""
    return unit_rms(x, eps) * (1.0 + w)


def norm_plain(x, w, eps):
    return unit_rms(x, eps) * w


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softmax_masked(scores: np.ndarray, visible: np.ndarray) -> np.ndarray:
    """Row-wise softmax over the entries where ``visible`` holds."""
    s = np.where(visible, scores, -np.inf)
    s = s - s.max(axis=-1, keepdims=True)
    e = np.where(visible, np.exp(s), 0.0)
    return e / e.sum(axis=-1, keepdims=True)


def window_mask(n: int, size: int) -> np.ndarray:
    i, j = np.arange(n)[:, None], np.arange(n)[None, :]
    return (i - j >= 0) & (i - j < size)


def chunk_mask(n: int, size: int) -> np.ndarray:
    i, j = np.arange(n)[:, None], np.arange(n)[None, :]
    return (j <= i) & (i // size == j // size)


def rotate_pairs(x: np.ndarray, dims: int, base: float) -> np.ndarray:
    """``x``: [tokens, heads, dim]; neighbours (2i, 2i+1) of the first ``dims`` elements of every
    head turn by ``position * base ** (-2i / dims)``."""
    out = x.copy()
    if dims == 0:
        return out
    pos = np.arange(x.shape[0], dtype=np.float64)[:, None, None]
    i = np.arange(dims // 2, dtype=np.float64)
    angle = pos * (base ** (-2.0 * i / dims))[None, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * np.cos(angle) - v * np.sin(angle)
    out[..., 1:dims:2] = v * np.cos(angle) + u * np.sin(angle)
    return out


def attention(h, w, prefix, m, eps):
    """Grouped heads, one norm over the whole q and the whole k projection, rotation, keys
    visible inside the query's chunk only."""
    n = h.shape[0]
    heads, groups, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = norm_plain(h @ w[prefix + "q"].T, w[prefix + "q.norm"], eps).reshape(n, heads, dim)
    k = norm_plain(h @ w[prefix + "k"].T, w[prefix + "k.norm"], eps).reshape(n, groups, dim)
    v = (h @ w[prefix + "v"].T).reshape(n, groups, vdim)
    q = rotate_pairs(q, m["rot"]["dims"], m["rot"]["base"])
    k = rotate_pairs(k, m["rot"]["dims"], m["rot"]["base"])
    visible = chunk_mask(n, m["mask"]["size"])
    out = np.zeros((n, heads, vdim))
    for head in range(heads):
        g = head // (heads // groups)
        p = softmax_masked(q[:, head] @ k[:, g].T * m["scale"], visible)
        out[:, head] = p @ v[:, g]
    return out.reshape(n, heads * vdim) @ w[prefix + "o"].T


def latent_attention(h, w, prefix, m, eps):
    """Queries and keys/values through normed latents, no positions, a sliding window, and a
    gate per head on the output."""
    n = h.shape[0]
    heads, dim, vdim = m["heads"], m["dim"], m["vdim"]
    cq = norm_plain(h @ w[prefix + "dq"].T, w[prefix + "dq.norm"], eps)
    q = (cq @ w[prefix + "uq"].T).reshape(n, heads, dim)
    c = norm_plain(h @ w[prefix + "dkv"].T, w[prefix + "dkv.norm"], eps)
    k = (c @ w[prefix + "uk"].T).reshape(n, heads, dim)
    v = (c @ w[prefix + "uv"].T).reshape(n, heads, vdim)
    gate = sigmoid(h @ w[prefix + "g"].T)
    visible = window_mask(n, m["mask"]["size"])
    out = np.zeros((n, heads, vdim))
    for head in range(heads):
        p = softmax_masked(q[:, head] @ k[:, head].T * m["scale"], visible)
        out[:, head] = (p @ v[:, head]) * gate[:, head:head + 1]
    return out.reshape(n, heads * vdim) @ w[prefix + "o"].T


def gated_expert(h, w, prefix):
    return (silu(h @ w[prefix + "gate"].T) * (h @ w[prefix + "up"].T)) @ w[prefix + "down"].T


def route(h, w, prefix, top, margins=None):
    """(experts [tokens, top], weights [tokens, top]): the largest logits, softmax over them.
    ``margins`` (a list) receives, per token, by how much the last chosen logit leads the first
    that is left out (infinite when every expert is chosen)."""
    z = h @ w[prefix + "router"].T + w[prefix + "router.b"]
    if margins is not None:
        ranked = -np.sort(-z, axis=-1)
        margins.append(ranked[:, top - 1] - ranked[:, top] if top < z.shape[1] else np.full(len(z), np.inf))
    order = np.argsort(-z, axis=-1, kind="stable")[:, :top]
    chosen = np.take_along_axis(z, order, axis=-1)
    e = np.exp(chosen - chosen.max(axis=-1, keepdims=True))
    return order, e / e.sum(axis=-1, keepdims=True)


def mixture(h, w, prefix, mlp, margins=None):
    experts, weights = route(h, w, prefix, mlp["router"]["top"], margins)
    out = np.zeros((h.shape[0], w[prefix + "e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for e, p in zip(experts[t], weights[t]):
            out[t] += p * gated_expert(h[t:t + 1], w, f"{prefix}e{e}.")[0]
    if mlp.get("shared") is not None:
        out += sigmoid(h @ w[prefix + "shared.sg"].T) * gated_expert(h, w, prefix + "shared.")
    return out


def layer_runs(config):
    """The order in which layers run: (layer, first of a pass that is not the first pass)."""
    count = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, False) for i in range(count)]
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    runs = [(i, False) for i in range(start)]
    for p in range(times):
        runs += [(i, p > 0 and i == start) for i in range(start, stop)]
    return runs + [(i, False) for i in range(stop, count)]


def forward(config, w, tokens, *, keep_layers: bool = False, margins=None):
    """Logits [tokens, vocab] of one whole sequence (and the stream after every layer run).
    ``margins`` (a list) receives every router's margins, see :func:`route`."""
    eps = config["norm"]["eps"]
    x = w["embed"][np.asarray(tokens)]
    embedded = x.copy()
    kept = []
    for index, again in layer_runs(config):
        layer = config["layers"][index]
        if again:
            x = x + embedded
        h = norm_around_zero(x, w[f"l{index}.norm1"], eps)
        mixer = {"attention": attention, "latent_attention": latent_attention}[layer["type"]]
        x = x + mixer(h, w, f"l{index}.mix.", layer["mixer"], eps)
        if layer.get("mlp") is not None:
            h = norm_around_zero(x, w[f"l{index}.norm2"], eps)
            x = x + mixture(h, w, f"l{index}.mlp.", layer["mlp"], margins)
        kept.append(x.copy())
    logits = norm_around_zero(x, w["final.norm"], eps) @ w["embed"].T
    cap = config.get("logit_softcap")
    if cap is not None:
        logits = cap * np.tanh(logits / cap)
    return (logits, np.stack(kept)) if keep_layers else logits
