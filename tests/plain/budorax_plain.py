"""A plain, slow implementation of the Budorax decoder in float64 numpy: whole sequences, no cache, no
batching, one function per mechanism.  It shares no code with the engine; the engine's tests compare
against it.

Notation: x [T, E] is the residual stream of one sequence, positions count from 0, linear weights are
[out, in] and applied as x @ W.T.  `cfg` is a mixer's (or feed-forward's) entry of config.json, `w` maps
the last part of a tensor's name ("q", "q.conv", "dkv.norm", "e3.gate", ...) to an array.
"""
from __future__ import annotations

import numpy as np


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.maximum(z, 0.0) + np.log1p(np.exp(-np.abs(z)))


def over_rms(x, eps):
    """x divided by the root of (its mean square along the last axis plus eps)."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def tanh_norm(x, weight, bias, alpha):
    """The norm that takes no mean and no variance: every element on its own."""
    return np.tanh(alpha * x) * weight + bias


# ---- positions ---------------------------------------------------------------------------------------------
def turn_pairs(x, positions, dims, base):
    """x [T, ..., D]: the first `dims` channels of the last axis turned by the token's position, channel 2i with
    channel 2i + 1, by the angle position * base^(-2i / dims); the other channels pass."""
    out = np.array(x, dtype=np.float64)
    T = x.shape[0]
    for i in range(dims // 2):
        angle = np.asarray(positions, dtype=np.float64) * base ** (-2.0 * i / dims)
        shape = (T,) + (1,) * (x.ndim - 2)
        c, s = np.cos(angle).reshape(shape), np.sin(angle).reshape(shape)
        a, b = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = a * c - b * s
        out[..., 2 * i + 1] = b * c + a * s
    return out


def seen_causal(T):
    i = np.arange(T)
    return i[None, :] <= i[:, None]


def seen_in_block(T, size):
    """Query i sees key j when j <= i and both lie in the same block of `size` positions counted from 0."""
    i = np.arange(T)
    return (i[None, :] <= i[:, None]) & ((i[None, :] // size) == (i[:, None] // size))


def masked_softmax(scores, seen):
    s = np.where(seen, scores, -np.inf)
    s = s - s.max(axis=-1, keepdims=True)
    e = np.exp(s)
    return e / e.sum(axis=-1, keepdims=True)


# ---- differential attention over blocks of positions ----------------------------------------------------
def differential_factor(w, diff):
    return np.exp(np.sum(w["lq1"] * w["lk1"])) - np.exp(np.sum(w["lq2"] * w["lk2"])) + diff


def block_differential_attention(x, w, cfg, eps):
    T = x.shape[0]
    H, G, D, V = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    pos = np.arange(T)
    q = (x @ w["q"].T).reshape(T, H, 2, D)
    k = (x @ w["k"].T).reshape(T, G, 2, D)
    v = (x @ w["v"].T).reshape(T, G, V)
    q = turn_pairs(q, pos, cfg["rot"]["dims"], cfg["rot"]["base"])
    k = turn_pairs(k, pos, cfg["rot"]["dims"], cfg["rot"]["base"])
    seen = seen_in_block(T, cfg["mask"]["size"])
    lam = differential_factor(w, cfg["diff"])
    heads = []
    for h in range(H):
        g = h // (H // G)
        maps = [masked_softmax(q[:, h, m] @ k[:, g, m].T * cfg["scale"], seen) @ v[:, g] for m in (0, 1)]
        o = maps[0] - lam * maps[1]
        heads.append(over_rms(o, eps) * (1.0 - cfg["diff"]))
    return np.concatenate(heads, axis=-1) @ w["o"].T


# ---- latent attention -----------------------------------------------------------------------------------
def latent_attention(x, w, cfg, eps):
    T = x.shape[0]
    H, D, R, V, rank = cfg["heads"], cfg["dim"], cfg["rot_dim"], cfg["vdim"], cfg["kv_rank"]
    pos = np.arange(T)
    base = cfg["rot"]["base"]
    cq = over_rms(x @ w["dq"].T, eps) * w["dq.norm"]
    q = (cq @ w["uq"].T).reshape(T, H, D + R)
    q_plain, q_turned = q[..., :D], turn_pairs(q[..., D:], pos, R, base)
    down = x @ w["dkv"].T
    c = over_rms(down[:, :rank], eps) * w["dkv.norm"]
    k_turned = turn_pairs(down[:, rank:], pos, R, base)          # one part for all heads
    k_plain = (c @ w["uk"].T).reshape(T, H, D)
    v = (c @ w["uv"].T).reshape(T, H, V)
    gate = sigmoid(x @ w["g"].T)                                  # [T, H]
    seen = seen_causal(T)
    heads = []
    for h in range(H):
        scores = (q_plain[:, h] @ k_plain[:, h].T + q_turned[:, h] @ k_turned.T) * cfg["scale"]
        heads.append(masked_softmax(scores, seen) @ v[:, h] * gate[:, h:h + 1])
    return np.concatenate(heads, axis=-1) @ w["o"].T


# ---- the gated delta rule -------------------------------------------------------------------------------
def short_convolution(x, taps):
    """x [T, C], taps [C, n]: y_t = sum_j taps[:, n - 1 - j] x_(t - j), zeros before the sequence."""
    T, n = x.shape[0], taps.shape[1]
    y = np.zeros_like(x)
    for j in range(min(n, T)):
        y[j:] += x[:T - j] * taps[:, n - 1 - j]
    return y


def delta_walk(q, k, v, beta, g):
    """q, k [T, dim], v [T, vdim], beta, g [T]: the state S [dim, vdim] from zero; the read sees the token's write."""
    T, V = v.shape
    S = np.zeros((q.shape[1], V))
    out = np.zeros((T, V))
    for t in range(T):
        S = g[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + np.outer(k[t], u)
        out[t] = S.T @ q[t]
    return out


def gated_delta(x, w, cfg, eps):
    T = x.shape[0]
    H, G, D, V = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    unit = lambda a: a / np.sqrt(np.sum(a * a, axis=-1, keepdims=True) + 1e-6)
    q = unit(silu(short_convolution(x @ w["q"].T, w["q.conv"])).reshape(T, G, D)) * D ** -0.5
    k = unit(silu(short_convolution(x @ w["k"].T, w["k.conv"])).reshape(T, G, D))
    v = silu(short_convolution(x @ w["v"].T, w["v.conv"])).reshape(T, H, V)
    beta = sigmoid(x @ w["b"].T)                                                          # [T, H]
    g = np.exp(-np.exp(w["A_log"]) * softplus(x @ w["a"].T + w["dt_bias"]))               # [T, H]
    gate = silu(x @ w["g"].T).reshape(T, H, V)
    heads = []
    for h in range(H):
        j = h // (H // G)
        o = delta_walk(q[:, j], k[:, j], v[:, h], beta[:, h], g[:, h])
        heads.append(over_rms(o, eps) * w["norm"] * gate[:, h])
    return np.concatenate(heads, axis=-1) @ w["o"].T


# ---- the feed-forward -----------------------------------------------------------------------------------
def choose_experts(x, w, router):
    """(the chosen experts [T, top], their weights [T, top]): sigmoid scores; the choice adds a correction a
    expert, the weights do not; the chosen scores over their sum, times the router's scale."""
    s = sigmoid(x @ w["router"].T)
    choice = s + w["correction"]
    ids = np.argsort(-choice, axis=-1, kind="stable")[:, :router["top"]]
    picked = np.take_along_axis(s, ids, axis=-1)
    return ids, picked / (picked.sum(axis=-1, keepdims=True) + 1e-20) * router["scale"]


def choice_margin(x, w, router, rounding=2.0 ** -8):
    """[T]: the gap between the last chosen and the first left-out choice score (infinite when all are chosen), in units
    of how far rounding every element of x by `rounding` (relative) may move a score.  A comparison with an engine that
    rounds may not rest on tokens whose margin is a small number."""
    s = sigmoid(x @ w["router"].T)
    moved = (s * (1.0 - s) * rounding * np.sqrt((x * x) @ (w["router"] ** 2).T)).max(axis=1) + 1e-300
    choice = -np.sort(-(s + w["correction"]), axis=-1)
    top = router["top"]
    gap = choice[:, top - 1] - choice[:, top] if top < choice.shape[1] else np.full(x.shape[0], np.inf)
    return gap / moved


def expert(x, w, e):
    return (silu(x @ w[f"e{e}.gate"].T) * (x @ w[f"e{e}.up"].T)) @ w[f"e{e}.down"].T


def expert_mixture(x, w, cfg):
    ids, weights = choose_experts(x, w, cfg["router"])
    out = np.zeros_like(x)
    for e in range(cfg["router"]["experts"]):
        rows, which = np.nonzero(ids == e)
        if len(rows):
            out[rows] += weights[rows, which][:, None] * expert(x[rows], w, e)
    return out


# ---- the model ------------------------------------------------------------------------------------------
MIXERS = {"attention": block_differential_attention, "latent_attention": latent_attention, "delta": gated_delta}


def part_weights(weights, prefix):
    return {name[len(prefix):]: np.asarray(t, dtype=np.float64) for name, t in weights.items() if name.startswith(prefix)}


def named_norm(weights, name, x):
    f = lambda n: np.asarray(weights[n], dtype=np.float64)
    return tanh_norm(x, f(name), f(name + ".b"), float(f(name + ".alpha")))


def run_order(config):
    """The layers in the order they run: [(layer, pass number, whether the pass starts here)]."""
    n = len(config["layers"])
    loop = config.get("loop") or {"start": 0, "stop": 0, "times": 1}
    order = [(i, 0, False) for i in range(loop["start"])]
    for p in range(loop["times"]):
        order += [(i, p, i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return order + [(i, 0, False) for i in range(loop["stop"], n)]


def forward(config, weights, tokens, streams=None, margins=None):
    """Logits [T, vocab] of one whole sequence.  `streams`, a list, receives the residual stream after every layer
    run; `margins`, a list, the routers' choice margins of every run."""
    eps = config["norm"]["eps"]
    table = np.asarray(weights["embed"], dtype=np.float64)
    x0 = table[np.asarray(tokens)]
    x = x0.copy()
    for i, p, starts in run_order(config):
        layer = config["layers"][i]
        if starts and p > 0:
            x = x + x0
        mixed = MIXERS[layer["type"]](named_norm(weights, f"l{i}.norm1", x), part_weights(weights, f"l{i}.mix."),
                                      layer["mixer"], eps)
        x = x + named_norm(weights, f"l{i}.norm1b", mixed)
        if layer.get("mlp") is not None:
            inner = named_norm(weights, f"l{i}.norm2", x)
            w = part_weights(weights, f"l{i}.mlp.")
            if margins is not None:
                margins.append(choice_margin(inner, w, layer["mlp"]["router"]))
            x = x + named_norm(weights, f"l{i}.norm2b", expert_mixture(inner, w, layer["mlp"]))
        if streams is not None:
            streams.append(x.copy())
    logits = named_norm(weights, "final.norm", x) @ table.T
    cap = config["logit_softcap"]
    return cap * np.tanh(logits / cap)


class PlainBudorax:
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

    def routing_margins(self, tokens):
        """[T]: every token's smallest choice margin over the layer runs, or None for a model without experts."""
        margins = []
        forward(self.cfg, self.tensors, tokens, margins=margins)
        return np.min(margins, axis=0) if margins else None

    def decisive(self, tokens, rng, least=40.0, tries=2000):
        """`tokens` with the token at every position whose routing is a close call (a margin below `least`) drawn
        again, until none is left (a position's margins depend on the tokens up to it only: the first close call of a
        pass is settled for good once its redraw is decisive, the later ones are drawn again along with it to save
        passes), so that an engine that rounds chooses the experts this file chooses."""
        tokens = list(tokens)
        vocab = self.tensors["embed"].shape[0]
        for _ in range(tries):
            margins = self.routing_margins(tokens)
            near = [] if margins is None else np.nonzero(margins < least)[0]
            if len(near) == 0:
                return tokens
            for at in near:
                tokens[int(at)] = int(rng.integers(0, vocab))
        raise ValueError("no decisive sequence found")

    def greedy(self, prompt, n):
        tokens, out = list(prompt), []
        for _ in range(n):
            t = int(np.argmax(self.logits(tokens, [len(tokens) - 1])[0]))
            out.append(t)
            tokens.append(t)
        return out
