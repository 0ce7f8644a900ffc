"""A plain, slow implementation of the Tigelorn decoder in float64 numpy: whole sequences, no cache, no
batching, one function per mechanism.  It shares no code with the engine; the engine's tests compare
against it.

Notation: x [T, E] is the residual stream of one sequence, positions count from 0, linear weights are
[out, in] and applied as x @ W.T.  `cfg` is a mixer's (or feed-forward's) entry of config.json, `w` maps
the last part of a tensor's name ("q", "q.conv", "left.q.b", "dkv.norm", ...) to an array.
"""
from __future__ import annotations

import numpy as np


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.maximum(z, 0.0) + np.log1p(np.exp(-np.abs(z)))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (z + 0.044715 * z ** 3)))


def rms(x, eps):
    """The root of (the mean square along the last axis plus eps)."""
    return np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def norm_around_zero(x, weight, eps):
    """RMS norm whose stored weight is the factor's distance from one."""
    return x / rms(x, eps) * (1.0 + weight)


def norm_plain(x, weight, eps):
    """RMS norm whose stored weight is the factor itself."""
    return x / rms(x, eps) * weight


# ---- the embedding ---------------------------------------------------------------------------------------
def bigram_rows(tokens, buckets, mul_prev, mul_cur):
    """The row of the pair table that every token of a sequence adds: a hash of (token before, token); the
    sequence's first token takes the table's last row."""
    rows = []
    for t, token in enumerate(tokens):
        rows.append(buckets if t == 0 else (int(tokens[t - 1]) * mul_prev + int(token) * mul_cur) % buckets)
    return np.asarray(rows, dtype=np.int64)


def embed(tokens, table, pairs, cfg):
    b = cfg["bigram"]
    return table[np.asarray(tokens)] + pairs[bigram_rows(tokens, b["buckets"], b["mul_prev"], b["mul_cur"])]


# ---- rotations --------------------------------------------------------------------------------------------
def yarn_frequencies(dims, base, scaling):
    """(frequency of every pair, factor on cosine and sine).  Without `scaling`: base^(-2 i / dims) and 1."""
    i = np.arange(dims // 2, dtype=np.float64)
    f = base ** (-2.0 * i / dims)
    if scaling is None:
        return f, 1.0
    factor, original = scaling["factor"], scaling["original"]

    def pair_of(turns):          # the pair whose wave makes `turns` turns over the original length
        return dims * np.log(original / (2.0 * np.pi * turns)) / (2.0 * np.log(base))
    lo = max(np.floor(pair_of(scaling["fast"])), 0)
    hi = min(np.ceil(pair_of(scaling["slow"])), dims - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * np.log(factor) + 1.0


def rotate(x, positions, dims, base, interleaved, scaling=None):
    """x [T, heads, D]: the first `dims` channels of every head turned by the token's position; pair i is the
    channels (2 i, 2 i + 1) when `interleaved`, else (i, i + dims / 2); the other channels pass."""
    half = dims // 2
    f, amp = yarn_frequencies(dims, base, scaling)
    angle = np.asarray(positions, dtype=np.float64)[:, None] * f[None, :]
    c, s = (amp * np.cos(angle))[:, None, :], (amp * np.sin(angle))[:, None, :]
    out = np.array(x, dtype=np.float64, copy=True)
    if interleaved:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    else:
        u, v = x[..., :half], x[..., half:dims]
        out[..., :half] = u * c - v * s
        out[..., half:dims] = v * c + u * s
    return out


# ---- softmax attention ------------------------------------------------------------------------------------
def seen_causal(T):
    p = np.arange(T)
    return p[None, :] <= p[:, None]


def seen_in_window(T, size):
    p = np.arange(T)
    d = p[:, None] - p[None, :]
    return (d >= 0) & (d < size)


def masked_softmax(scores, seen):
    s = np.where(seen, scores, -np.inf)
    p = np.exp(s - s.max(axis=1, keepdims=True))
    return p / p.sum(axis=1, keepdims=True)


def window_attention(x, w, cfg, eps):
    """Grouped-query attention over a sliding window: biased q/k/v, a rotation of a head's first channels in
    split-half pairs, then q and k over their root mean square per head (no weight), a gate on the heads."""
    T = x.shape[0]
    H, G, D, V = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    q = (x @ w["q"].T + w["q.b"]).reshape(T, H, D)
    k = (x @ w["k"].T + w["k.b"]).reshape(T, G, D)
    v = (x @ w["v"].T + w["v.b"]).reshape(T, G, V)
    pos = np.arange(T)
    q = rotate(q, pos, cfg["rot"]["dims"], cfg["rot"]["base"], interleaved=False)
    k = rotate(k, pos, cfg["rot"]["dims"], cfg["rot"]["base"], interleaved=False)
    q, k = q / rms(q, eps), k / rms(k, eps)
    seen = seen_in_window(T, cfg["mask"]["size"])
    heads = []
    for head in range(H):
        g = head // (H // G)
        heads.append(masked_softmax((q[:, head] @ k[:, g].T) * cfg["scale"], seen) @ v[:, g])
    return (np.concatenate(heads, axis=1) * sigmoid(x @ w["g"].T)) @ w["o"].T


def latent_attention(x, w, cfg, eps):
    """Queries through a normed latent; keys and values of all heads from one normed latent a token plus one
    rotated key part shared by the heads (interleaved pairs, stretched frequencies); causal."""
    T = x.shape[0]
    H, D, R, V, C = cfg["heads"], cfg["dim"], cfg["rot_dim"], cfg["vdim"], cfg["kv_rank"]
    rot = cfg["rot"]
    q = (norm_plain(x @ w["dq"].T, w["dq.norm"], eps) @ w["uq"].T).reshape(T, H, D + R)
    down = x @ w["dkv"].T
    latent = norm_plain(down[:, :C], w["dkv.norm"], eps)
    pos = np.arange(T)
    q_rot = rotate(q[..., D:], pos, rot["dims"], rot["base"], True, rot.get("scaling"))
    k_rot = rotate(down[:, None, C:], pos, rot["dims"], rot["base"], True, rot.get("scaling"))[:, 0]
    k_plain = (latent @ w["uk"].T).reshape(T, H, D)
    v = (latent @ w["uv"].T).reshape(T, H, V)
    seen = seen_causal(T)
    heads = []
    for head in range(H):
        s = (q[:, head, :D] @ k_plain[:, head].T + q_rot[:, head] @ k_rot.T) * cfg["scale"]
        heads.append(masked_softmax(s, seen) @ v[:, head])
    return np.concatenate(heads, axis=1) @ w["o"].T


# ---- recurrent mixers -------------------------------------------------------------------------------------
def short_convolution(x, taps):
    """x [T, C], taps [C, K]: y[t, c] = sum_j taps[c, j] x[t - (K - 1 - j), c], zeros before the start."""
    T, K = x.shape[0], taps.shape[1]
    padded = np.concatenate([np.zeros((K - 1, x.shape[1])), x], axis=0)
    y = np.zeros_like(x, dtype=np.float64)
    for j in range(K):
        y += padded[j:j + T] * taps[:, j][None, :]
    return y


def decayed_sum_attention(x, w, cfg, eps):
    """Linear attention with one constant decay a head: S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t on
    silu'd projections; the heads side by side normed as one row, gated, projected."""
    T = x.shape[0]
    H, D, V = cfg["heads"], cfg["dim"], cfg["vdim"]
    q, k = silu(x @ w["q"].T).reshape(T, H, D), silu(x @ w["k"].T).reshape(T, H, D)
    v = silu(x @ w["v"].T).reshape(T, H, V)
    out = np.zeros((T, H, V))
    for head in range(H):
        S = np.zeros((D, V))
        for t in range(T):
            S = cfg["decay"][head] * S + np.outer(k[t, head], v[t, head])
            out[t, head] = S.T @ q[t, head]
    o = norm_plain(out.reshape(T, H * V), w["norm"], eps)
    return (o * sigmoid(x @ w["g"].T)) @ w["o"].T


def two_mixers(x, w, cfg, eps):
    sub = lambda side: {name[len(side) + 1:]: value for name, value in w.items() if name.startswith(side + ".")}
    return (cfg["left_scale"] * window_attention(x, sub("left"), cfg["left"], eps)
            + cfg["right_scale"] * decayed_sum_attention(x, sub("right"), cfg["right"], eps))


def delta_rule(q, k, v, beta, g):
    """One head.  q, k [T, D] (unit vectors, q scaled), v [T, V], beta [T], g [T, D] decays of the key channels:
    S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q."""
    T, D = q.shape
    S = np.zeros((D, v.shape[1]))
    out = np.zeros((T, v.shape[1]))
    for t in range(T):
        S = g[t][:, None] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + np.outer(k[t], u)
        out[t] = S.T @ q[t]
    return out


def channel_delta(x, w, cfg, eps):
    """Gated delta rule with a decay per key channel: q/k/v through a short causal convolution and silu, q and k
    unit vectors per head, the write strength beta and the decays from the input, each head's read-out normed
    over its value channels, gated and projected."""
    T = x.shape[0]
    H, G, D, V = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    q = silu(short_convolution(x @ w["q"].T, w["q.conv"])).reshape(T, G, D)
    k = silu(short_convolution(x @ w["k"].T, w["k.conv"])).reshape(T, G, D)
    v = silu(short_convolution(x @ w["v"].T, w["v.conv"])).reshape(T, H, V)
    q = q / np.sqrt((q * q).sum(axis=-1, keepdims=True) + 1e-6) * D ** -0.5
    k = k / np.sqrt((k * k).sum(axis=-1, keepdims=True) + 1e-6)
    beta = sigmoid(x @ w["b"].T)                                                 # [T, H]
    rate = softplus((x @ w["a1"].T) @ w["a2"].T + w["dt_bias"]).reshape(T, H, D)
    g = np.exp(-np.exp(w["A_log"])[None, :, None] * rate)
    gate = sigmoid((x @ w["g1"].T) @ w["g2"].T).reshape(T, H, V)
    out = np.zeros((T, H, V))
    for head in range(H):
        kv = head // (H // G)
        out[:, head] = delta_rule(q[:, kv], k[:, kv], v[:, head], beta[:, head], g[:, head])
    out = out / rms(out, eps) * w["norm"] * gate
    return out.reshape(T, H * V) @ w["o"].T


def gated_ffn(x, w):
    return (gelu_tanh(x @ w["gate"].T) * (x @ w["up"].T)) @ w["down"].T


MIXERS = {"parallel": two_mixers, "channel_delta": channel_delta, "latent_attention": latent_attention}


def layer_weights(weights, layer, part):
    prefix = f"l{layer}.{part}."
    return {name[len(prefix):]: value for name, value in weights.items() if name.startswith(prefix)}


def forward(config, weights, tokens, streams=None):
    """Logits [T, vocab] of one sequence from position 0.  `weights`: {tensor name: float64 array}.
    `streams`, a list, receives the residual stream after every layer."""
    eps = config["norm"]["eps"]
    x = embed(tokens, weights["embed"], weights["bigram"], config["embedding"])
    for i, layer in enumerate(config["layers"]):
        own = layer.get("weights_of", i)                   # a layer may run with another layer's tensors
        mixed = MIXERS[layer["type"]](norm_around_zero(x, weights[f"l{own}.norm1"], eps),
                                      layer_weights(weights, own, "mix"), layer["mixer"], eps)
        x = x + mixed
        if layer.get("mlp") is not None:
            x = x + gated_ffn(norm_around_zero(x, weights[f"l{own}.norm2"], eps), layer_weights(weights, own, "mlp"))
        if streams is not None:
            streams.append(x.copy())
    return norm_around_zero(x, weights["final.norm"], eps) @ weights["embed"].T


class PlainTigelorn:
    """A model folder (config.json, model.safetensors) run by the functions above."""

    def __init__(self, folder):
        import json
        import os

        import torch
        from safetensors.torch import load_file
        with open(os.path.join(folder, "config.json")) as f:
            self.cfg = json.load(f)
        self.tensors = {n: (t.to(torch.float64) if t.dtype.is_floating_point else t).numpy()
                        for n, t in load_file(os.path.join(folder, "model.safetensors")).items()}

    def logits(self, tokens, want=None):
        rows = forward(self.cfg, self.tensors, tokens)
        return rows if want is None else rows[np.asarray(want, dtype=np.int64)]

    def streams(self, tokens):
        out = []
        forward(self.cfg, self.tensors, tokens, streams=out)
        return np.stack(out)

    def greedy(self, prompt, n):
        tokens, out = list(prompt), []
        for _ in range(n):
            t = int(np.argmax(self.logits(tokens, [len(tokens) - 1])[0]))
            out.append(t)
            tokens.append(t)
        return out
