"""Plain, slow restatement of the Lenuzen design (test infrastructure only).

One function per mechanism, float64 numpy, whole sequences at once (no cache, no
state object): position t of every function sees exactly the positions its mask
allows. Nothing here is shared with the product path; the tests compare the HIP
engine against these functions on small random models.

A model is (cfg, w): cfg the parsed config.json dict, w a dict name -> float64
array under the checkpoint's tensor names.
"""

from __future__ import annotations

import math

import numpy as np

F = np.float64


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (z + 0.044715 * z**3)))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def unit_rms(x, eps):
    """x divided by its root mean square over the last axis (eps inside the root)."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def layer_norm(x, w, eps):
    """Mean-subtracting norm with a weight and no bias."""
    d = x - np.mean(x, axis=-1, keepdims=True)
    return d / np.sqrt(np.mean(d * d, axis=-1, keepdims=True) + eps) * w


def embed(cfg, w, tokens):
    return w["embed"][np.asarray(tokens)] * cfg["embedding"]["scale"]


def rotary_table(rot, positions):
    """cos, sin [T, dims / 2] of the scaled rotary angles."""
    dims, base = rot["dims"], rot["base"]
    half = dims // 2
    f = np.array([base ** (-2.0 * i / dims) for i in range(half)], F)
    mag = 1.0
    sc = rot.get("scaling")
    if sc:
        factor, orig = sc["factor"], sc["original"]

        def turn(t):
            return dims * math.log(orig / (2.0 * math.pi * t)) / (2.0 * math.log(base))

        lo = max(math.floor(turn(sc["fast"])), 0)
        hi = min(math.ceil(turn(sc["slow"])), dims - 1)
        ramp = np.clip((np.arange(half, dtype=F) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    ang = np.asarray(positions, F)[:, None] * f[None, :]
    return np.cos(ang) * mag, np.sin(ang) * mag


def rotate(x, rot, positions):
    """x [T, heads, dim]: the first rot.dims entries of every head turn in interleaved
    pairs (2i, 2i + 1), the rest pass."""
    dims = rot["dims"]
    cos, sin = rotary_table(rot, positions)
    out = x.copy()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    c, s = cos[:, None, :], sin[:, None, :]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def visible(kind, size, T):
    """mask[i, j]: position i sees position j."""
    i = np.arange(T)[:, None]
    j = np.arange(T)[None, :]
    if kind == "window":
        return (j <= i) & (i - j < size)
    if kind == "chunk":
        return (j <= i) & (i // size == j // size)
    return j <= i


def softmax_rows(s, mask, sink):
    """Softmax over the visible keys of every row; sink: one more key of score 0 and no value."""
    s = np.where(mask, s, -np.inf)
    m = np.max(s, axis=-1, keepdims=True)
    if sink:
        m = np.maximum(m, 0.0)
    e = np.where(mask, np.exp(s - m), 0.0)
    den = e.sum(axis=-1, keepdims=True)
    if sink:
        den = den + np.exp(-m)
    return e / den


def attention_core(q, k, v, scale, mask, temp=None, talk=None, sink=False):
    """q [T, H, D], k [T, G, D], v [T, G, V] -> (out [T, H, V], weights [H, T, T])."""
    T, H, _ = q.shape
    G = k.shape[1]
    rep = H // G
    s = np.stack([q[:, h] @ k[:, h // rep].T for h in range(H)]) * scale
    if temp is not None:
        s = s * temp[:, None, None]
    if talk is not None:
        s = np.einsum("hg,gij->hij", talk, s)
    p = softmax_rows(s, mask[None], sink)
    out = np.stack([p[h] @ v[:, h // rep] for h in range(H)], axis=1)
    return out, p


def mixer_attention(cfg, w, pre, h, m, positions=None, weights_out=None):
    """Biased projections, rotation, per-head unit-rms queries / keys / values, per-head
    temperature, sliding window, plain softmax, per-head sigmoid output gate."""
    T = h.shape[0]
    eps = cfg["norm"]["eps"]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = np.arange(T) if positions is None else positions
    q = (h @ w[pre + "q"].T + w[pre + "q.b"]).reshape(T, H, D)
    k = (h @ w[pre + "k"].T + w[pre + "k.b"]).reshape(T, G, D)
    v = (h @ w[pre + "v"].T + w[pre + "v.b"]).reshape(T, G, V)
    q = unit_rms(rotate(q, m["rot"], pos), eps)
    k = unit_rms(rotate(k, m["rot"], pos), eps)
    v = unit_rms(v, eps)
    mask = visible("window", m["mask"]["size"], T)
    o, p = attention_core(q, k, v, m["scale"], mask, temp=w[pre + "temp"])
    if weights_out is not None:
        weights_out.append(p)
    gate = sigmoid(h @ w[pre + "g"].T)
    o = o * gate[:, :, None]
    return o.reshape(T, H * V) @ w[pre + "o"].T


def mixer_attention_2(cfg, w, pre, h, m, positions=None, weights_out=None):
    """Whole-projection rms norm of queries and keys (weighted) before rotation, scores
    mixed across heads, chunked mask, softmax with a zero-score sink."""
    T = h.shape[0]
    eps = cfg["norm"]["eps"]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = np.arange(T) if positions is None else positions
    q = unit_rms(h @ w[pre + "q"].T, eps) * w[pre + "q.norm"]
    k = unit_rms(h @ w[pre + "k"].T, eps) * w[pre + "k.norm"]
    v = (h @ w[pre + "v"].T).reshape(T, G, V)
    q = rotate(q.reshape(T, H, D), m["rot"], pos)
    k = rotate(k.reshape(T, G, D), m["rot"], pos)
    mask = visible("chunk", m["mask"]["size"], T)
    o, p = attention_core(q, k, v, m["scale"], mask, talk=w[pre + "talk"], sink=True)
    if weights_out is not None:
        weights_out.append(p)
    return o.reshape(T, H * V) @ w[pre + "o"].T


MIXERS = {"attention": mixer_attention, "attention_2": mixer_attention_2}


def dense_ff(w, pre, h):
    return gelu_tanh(h @ w[pre + "up"].T) @ w[pre + "down"].T


def forward(cfg, w, tokens, layers_out=None, weights_out=None):
    """Logits [T, vocab] of a whole sequence; layers_out (a list) receives the residual
    stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = embed(cfg, w, tokens)
    for i, e in enumerate(cfg["layers"]):
        p = f"l{i}."
        x = x + layer_norm(MIXERS[e["type"]](cfg, w, p + "mix.", x, e["mixer"], weights_out=weights_out),
                           w[p + "norm1"], eps)
        if e.get("mlp"):
            x = x + layer_norm(dense_ff(w, p + "mlp.", x), w[p + "norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.copy())
    y = layer_norm(x, w["final.norm"], eps)
    return (y @ w["embed"].T) * cfg["logit_scale"]
