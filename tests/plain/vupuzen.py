"""A plain, slow implementation of the Vupuzen decoder: whole sequences, no cache, numpy
float64, one function per mechanism.  It shares no code with ``pylon_amd`` and is the
oracle of the tests.

The design in this file's notation.  With ``rms(x) = sqrt(mean(x^2) + eps)``:

* a layer:  ``x += b1 * m / rms(m)`` with ``m = mixer(h + conv(h))``, ``h = a1 * x / rms(x)``;
  then, if it has a feed-forward, ``x += b2 * f / rms(f)`` with ``f = ff(a2 * x / rms(x))``;
  ``a1, b1, a2, b2`` are single numbers;
* ``conv(h)[t] = sum_j w[:, j] * h[t - taps + 1 + j]`` per channel, zero before the start;
* attention: ``s_ij = scale * q_i.k_j + rel[bucket(i - j), head]``, weights
  ``exp(s_ij) / (1 + sum_j' exp(s_ij'))`` over ``j <= i``, grouped key/value heads, keys of
  ``dim`` and values of ``vdim`` elements, no rotation;
* retention: rotary q and k (first ``dims`` elements of a head, pairs ``(i, i + dims/2)``),
  ``k *= dim ** -0.5``, ``S_t = decay_h S_{t-1} + k_t v_t^T``, ``o_t = S_t^T q_t``,
  ``o / rms(o)`` per head, times ``silu(W_g h)``, then ``W_o``;
* feed-forward: ``g = min(W_gate h, L)``, ``u = clip(W_up h, -L, L)``,
  ``W_down (g * sigmoid(1.702 g) * (u + 1))``;
* output: ``head (c * x / rms(x)) * logit_scale``.

Weights come as a dict from tensor name to array, the configuration as the raw content of
config.json.
"""
from __future__ import annotations

import math
from typing import List, Mapping, Optional, Sequence

import numpy as np

F = np.float64


def scalar_rms_norm(x: np.ndarray, gain, eps: float) -> np.ndarray:
    """``gain * x / sqrt(mean(x^2) + eps)`` over the last axis; ``gain`` is one number."""
    x = np.asarray(x, dtype=F)
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * float(gain)


def causal_conv(h: np.ndarray, w: np.ndarray) -> np.ndarray:
    """``h``: [T, width]; ``w``: [width, taps].  Tap ``j`` weighs the input ``taps - 1 - j``
    steps back; the last tap weighs the current input."""
    tokens, _ = h.shape
    taps = w.shape[1]
    out = np.zeros_like(h, dtype=F)
    for t in range(tokens):
        for j in range(taps):
            src = t - taps + 1 + j
            if src >= 0:
                out[t] += w[:, j] * h[src]
    return out


def distance_bucket(n: int, rows: int, far: float) -> int:
    """Row of the bias table for a key ``n`` tokens behind its query: the first half of the
    rows take distances one by one, the second half spreads logarithmically up to ``far``;
    everything beyond lands in the last row."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def sink_softmax_attention(q, k, v, rel, scale: float, far: float) -> np.ndarray:
    """q: [H, T, dim]; k: [G, T, dim]; v: [G, T, vdim]; rel: [rows, H].  Returns [H, T, vdim]."""
    heads, tokens, _ = q.shape
    group = heads // k.shape[0]
    rows = rel.shape[0]
    bucket = np.array([distance_bucket(n, rows, far) for n in range(tokens)], dtype=np.int64)
    out = np.zeros((heads, tokens, v.shape[-1]), dtype=F)
    for h in range(heads):
        kh, vh = k[h // group], v[h // group]
        for i in range(tokens):
            s = (kh[: i + 1] @ q[h, i]) * scale + rel[bucket[i - np.arange(i + 1)], h]
            top = max(float(s.max()), 0.0)
            e = np.exp(s - top)
            out[h, i] = (e @ vh[: i + 1]) / (math.exp(-top) + e.sum())
    return out


def rotate_half_layout(x: np.ndarray, positions: Sequence[int], dims: int, base: float) -> np.ndarray:
    """x: [H, T, dim]; rotates the first ``dims`` elements of every head.  Frequencies and
    angles are formed in float32, as a 32-bit implementation forms them."""
    half = dims // 2
    index = np.arange(half, dtype=np.float32)
    freq = np.power(np.float32(base), -(np.float32(2.0) * index / np.float32(dims)), dtype=np.float32)
    angle = (np.asarray(positions, dtype=np.float32)[:, None] * freq[None, :]).astype(np.float32).astype(F)
    cos, sin = np.cos(angle)[None], np.sin(angle)[None]
    out = np.array(x, dtype=F, copy=True)
    u, w = x[..., :half], x[..., half:dims]
    out[..., :half] = u * cos - w * sin
    out[..., half:dims] = w * cos + u * sin
    return out


def retention(q, k, v, decay: Sequence[float], eps: float, state: Optional[np.ndarray] = None):
    """q, k: [H, T, dim] (rotated, k scaled); v: [H, T, vdim].  Returns (normalised o
    [H, T, vdim], final state [H, dim, vdim])."""
    heads, tokens, dim = q.shape
    vdim = v.shape[-1]
    s = np.zeros((heads, dim, vdim), dtype=F) if state is None else np.array(state, dtype=F)
    out = np.zeros((heads, tokens, vdim), dtype=F)
    for t in range(tokens):
        for h in range(heads):
            s[h] = decay[h] * s[h] + np.outer(k[h, t], v[h, t])
            o = s[h].T @ q[h, t]
            out[h, t] = o / math.sqrt(float(np.mean(o * o)) + eps)
    return out, s


def silu(x):
    return x / (1.0 + np.exp(-x))


def capped_gated_mlp(h, w_gate, w_up, w_down, limit: float) -> np.ndarray:
    g = np.minimum(h @ w_gate.T, limit)
    u = np.clip(h @ w_up.T, -limit, limit)
    return (g / (1.0 + np.exp(-1.702 * g)) * (u + 1.0)) @ w_down.T


def attention_mixer(h, w: Mapping[str, np.ndarray], p: str, m: Mapping) -> np.ndarray:
    tokens = h.shape[0]
    heads, groups, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).reshape(tokens, heads, dim).transpose(1, 0, 2)
    k = (h @ w[p + "k"].T).reshape(tokens, groups, dim).transpose(1, 0, 2)
    v = (h @ w[p + "v"].T).reshape(tokens, groups, vdim).transpose(1, 0, 2)
    o = sink_softmax_attention(q, k, v, w[p + "rel"], float(m["scale"]), float(m["bias_max"]))
    return o.transpose(1, 0, 2).reshape(tokens, heads * vdim) @ w[p + "o"].T


def retention_mixer(h, w: Mapping[str, np.ndarray], p: str, m: Mapping, eps: float) -> np.ndarray:
    tokens = h.shape[0]
    heads, dim, vdim = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).reshape(tokens, heads, dim).transpose(1, 0, 2)
    k = (h @ w[p + "k"].T).reshape(tokens, heads, dim).transpose(1, 0, 2)
    v = (h @ w[p + "v"].T).reshape(tokens, heads, vdim).transpose(1, 0, 2)
    positions = np.arange(tokens)
    q = rotate_half_layout(q, positions, m["rot"]["dims"], float(m["rot"]["base"]))
    k = rotate_half_layout(k, positions, m["rot"]["dims"], float(m["rot"]["base"])) * dim ** -0.5
    o, _ = retention(q, k, v, m["decay"], eps)
    gate = silu(h @ w[p + "g"].T)
    return (o.transpose(1, 0, 2).reshape(tokens, heads * vdim) * gate) @ w[p + "o"].T


def forward(weights: Mapping[str, np.ndarray], cfg: Mapping, tokens: Sequence[int],
            residuals: Optional[List[np.ndarray]] = None) -> np.ndarray:
    """Logits [T, vocab] of one whole sequence.  ``residuals`` (a list) receives the stream
    after every layer run."""
    w = {name: np.asarray(t, dtype=F) for name, t in weights.items()}
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][np.asarray(tokens)]
    for index, entry in enumerate(cfg["layers"]):
        owner = entry.get("weights_of", index)
        p = f"l{owner}."
        h = scalar_rms_norm(x, w[p + "norm1"], eps)
        h = h + causal_conv(h, w[p + "canon1"])
        if entry["type"] == "attention":
            mixed = attention_mixer(h, w, p + "mix.", entry["mixer"])
        elif entry["type"] == "retention":
            mixed = retention_mixer(h, w, p + "mix.", entry["mixer"], eps)
        else:
            raise ValueError(f"unknown layer type {entry['type']!r}")
        x = x + scalar_rms_norm(mixed, w[p + "norm1b"], eps)
        if entry.get("mlp") is not None:
            h = scalar_rms_norm(x, w[p + "norm2"], eps)
            f = capped_gated_mlp(h, w[p + "mlp.gate"], w[p + "mlp.up"], w[p + "mlp.down"], float(entry["mlp"]["limit"]))
            x = x + scalar_rms_norm(f, w[p + "norm2b"], eps)
        if residuals is not None:
            residuals.append(x.copy())
    x = scalar_rms_norm(x, w["final.norm"], eps)
    return (x @ w["head"].T) * float(cfg["logit_scale"])


def greedy(logits_row: np.ndarray) -> int:
    return int(np.argmax(logits_row))
