"""Plain, slow restatement of the Sinulorn design (test infrastructure only).

One function per mechanism, float64 numpy, whole sequences at once (no cache,
no state object): position t of every function sees exactly positions 0..t.
Nothing here is shared with the product path; the tests compare the HIP
engine against these functions on small random models.

A model is (cfg, w): cfg the parsed config.json dict, w a dict name -> float64
array under the checkpoint's tensor names.
"""

from __future__ import annotations

import numpy as np

F = np.float64


def rms_norm(x, w, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (z + 0.044715 * z**3)))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def embed(cfg, w, tokens):
    """Scaled embedding rows plus the interleaved sin / cos position vector."""
    width = cfg["width"]
    x = w["embed"][np.asarray(tokens)] * cfg["embedding"]["scale"]
    p = np.arange(len(tokens), dtype=F)[:, None]
    i = np.arange(width // 2, dtype=F)[None, :]
    ang = p * 10000.0 ** (-2.0 * i / width)
    pe = np.zeros((len(tokens), width), F)
    pe[:, 0::2] = np.sin(ang)
    pe[:, 1::2] = np.cos(ang)
    return x + pe


def causal_conv(x, taps_w, bias=None):
    """Per-channel causal convolution over time: taps_w [channels, taps], the last
    column multiplies the current token, zeros before the start."""
    T, C = x.shape
    K = taps_w.shape[1]
    xp = np.concatenate([np.zeros((K - 1, C), F), x], axis=0)
    out = np.zeros((T, C), F)
    for j in range(K):
        out += xp[j:j + T] * taps_w[:, j][None, :]
    if bias is not None:
        out = out + bias
    return out


def latent(cfg, w, pre, h, m, eps):
    """The normalised key/value latent of one latent-attention layer: [T, kv_rank]."""
    return rms_norm(h @ w[pre + "dkv"].T, w[pre + "dkv.norm"], eps)


def attention_weights(cfg, w, pre, h, m, eps, c):
    """Softmax weights [heads, T, T] of a latent-attention layer (row t over keys j <= t)."""
    T = h.shape[0]
    H, D = m["heads"], m["dim"]
    cq = rms_norm(h @ w[pre + "dq"].T, w[pre + "dq.norm"], eps)
    q = (cq @ w[pre + "uq"].T).reshape(T, H, D)
    k = (c @ w[pre + "uk"].T).reshape(T, H, D)
    mask = np.tril(np.ones((T, T), bool))
    P = np.zeros((H, T, T), F)
    for hh in range(H):
        s = (q[:, hh] @ k[:, hh].T) * m["scale"]
        s = np.where(mask, s, -np.inf)
        s = s - s.max(axis=1, keepdims=True)
        p = np.exp(s)
        P[hh] = p / p.sum(axis=1, keepdims=True)
    return P


def latent_attention(cfg, w, pre, h, m, eps, c):
    """Causal softmax attention whose keys and values are up-projections of the
    latent c [T, kv_rank] (this layer's own or another layer's)."""
    T = h.shape[0]
    H, V = m["heads"], m["vdim"]
    P = attention_weights(cfg, w, pre, h, m, eps, c)
    v = (c @ w[pre + "uv"].T).reshape(T, H, V)
    out = np.stack([P[hh] @ v[:, hh] for hh in range(H)], axis=1)
    return out.reshape(T, H * V) @ w[pre + "o"].T


def rglru(cfg, w, pre, h, m):
    """Gated recurrent block: a gelu branch times a real-gated linear recurrence over
    the convolved second branch."""
    T = h.shape[0]
    W, B = m["width"], m["blocks"]
    y = gelu_tanh(h @ w[pre + "y"].T + w[pre + "y.b"])
    u = causal_conv(h @ w[pre + "x"].T + w[pre + "x.b"], w[pre + "conv"], w[pre + "conv.b"])
    bs = W // B
    ub = u.reshape(T, B, bs)
    r = sigmoid(np.einsum("boi,tbi->tbo", w[pre + "ra"], ub) + w[pre + "ra.b"]).reshape(T, W)
    i = sigmoid(np.einsum("boi,tbi->tbo", w[pre + "ri"], ub) + w[pre + "ri.b"]).reshape(T, W)
    log_a = -8.0 * r * softplus(w[pre + "lam"])
    a = np.exp(log_a)
    S = np.zeros(W, F)
    out = np.zeros((T, W), F)
    for t in range(T):
        S = a[t] * S + np.sqrt(1.0 - a[t] ** 2) * i[t] * u[t]
        out[t] = S
    return (out * y) @ w[pre + "o"].T


def delta(cfg, w, pre, h, m, eps):
    """Gated delta rule: per head a [dim, vdim] state, decayed, corrected towards the
    current value along the current key, then read with the query."""
    T = h.shape[0]
    H, KH, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(h @ w[pre + "q"].T, w[pre + "q.conv"])).reshape(T, KH, D)
    k = silu(causal_conv(h @ w[pre + "k"].T, w[pre + "k.conv"])).reshape(T, KH, D)
    v = silu(causal_conv(h @ w[pre + "v"].T, w[pre + "v.conv"])).reshape(T, H, V)
    q = q / np.sqrt(np.sum(q * q, axis=-1, keepdims=True) + 1e-6) * D ** -0.5
    k = k / np.sqrt(np.sum(k * k, axis=-1, keepdims=True) + 1e-6)
    beta = sigmoid(h @ w[pre + "b"].T)
    g = np.exp(-np.exp(w[pre + "A_log"]) * softplus(h @ w[pre + "a"].T + w[pre + "dt_bias"]))
    gate = silu(h @ w[pre + "g"].T).reshape(T, H, V)
    rep = H // KH
    o = np.zeros((T, H, V), F)
    for hh in range(H):
        kh = hh // rep
        S = np.zeros((D, V), F)
        for t in range(T):
            S = g[t, hh] * S
            u = beta[t, hh] * (v[t, hh] - S.T @ k[t, kh])
            S = S + np.outer(k[t, kh], u)
            o[t, hh] = S.T @ q[t, kh]
    o = o / np.sqrt(np.mean(o * o, axis=-1, keepdims=True) + eps) * w[pre + "norm"] * gate
    return o.reshape(T, H * V) @ w[pre + "o"].T


def dense_ff(w, pre, h):
    return (gelu_tanh(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def expert_ff(w, pre, h, limit):
    g = np.minimum(h @ w[pre + "gate"].T, limit)
    u = np.clip(h @ w[pre + "up"].T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w[pre + "down"].T


def route(w, pre, h, r):
    """Chosen experts and their weights per token: softmax scores, the best
    groups.keep groups by their best score, the top experts among those."""
    E, top = r["experts"], r["top"]
    z = h @ w[pre + "router"].T
    z = z - z.max(axis=1, keepdims=True)
    s = np.exp(z)
    s /= s.sum(axis=1, keepdims=True)
    G, keep = r["groups"]["count"], r["groups"]["keep"]
    gs = s.reshape(-1, G, E // G).max(axis=2)
    order = np.argsort(-gs, axis=1, kind="stable")[:, :keep]
    allowed = np.zeros((h.shape[0], G), bool)
    np.put_along_axis(allowed, order, True, axis=1)
    masked = np.where(np.repeat(allowed, E // G, axis=1), s, -1.0)
    idx = np.argsort(-masked, axis=1, kind="stable")[:, :top]
    return idx, np.take_along_axis(s, idx, axis=1) * r["scale"]


def moe_ff(w, pre, h, mlp):
    idx, wt = route(w, pre, h, mlp["router"])
    out = np.zeros((h.shape[0], w[pre + "e0.down"].shape[0]), F)
    for e in range(mlp["router"]["experts"]):
        for slot in range(idx.shape[1]):
            rows = np.nonzero(idx[:, slot] == e)[0]
            if len(rows):
                out[rows] += wt[rows, slot][:, None] * expert_ff(w, f"{pre}e{e}.", h[rows], mlp["expert"]["limit"])
    if mlp.get("shared"):
        sg = sigmoid(h @ w[pre + "shared.sg"].T)
        out += sg * expert_ff(w, pre + "shared.", h, mlp["shared"]["limit"])
    return out


def forward(cfg, w, tokens, layers_out=None):
    """Logits [T, vocab] of one sequence; layers_out (a list) receives the residual
    stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = embed(cfg, w, tokens)
    latents = {}
    for li, layer in enumerate(cfg["layers"]):
        p = f"l{li}."
        m = layer["mixer"]
        h = rms_norm(x, w[p + "norm1"], eps)
        if layer["type"] == "latent_attention":
            src = m.get("kv_from")
            if src is None:
                latents[li] = latent(cfg, w, p + "mix.", h, m, eps)
                src = li
            y = latent_attention(cfg, w, p + "mix.", h, m, eps, latents[src])
        elif layer["type"] == "rglru":
            y = rglru(cfg, w, p + "mix.", h, m)
        elif layer["type"] == "delta":
            y = delta(cfg, w, p + "mix.", h, m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + rms_norm(y, w[p + "norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp:
            h = rms_norm(x, w[p + "norm2"], eps)
            y = dense_ff(w, p + "mlp.", h) if mlp["kind"] == "dense" else moe_ff(w, p + "mlp.", h, mlp)
            x = x + rms_norm(y, w[p + "norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.copy())
    return rms_norm(x, w["final.norm"], eps) @ w["head"].T
