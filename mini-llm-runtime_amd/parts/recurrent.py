"""Mixers that keep a state of fixed size per request instead of keys and values: gated linear attention,
Mamba-2, linear attention with a constant decay a head, and the gated delta rule.  The first three run the same
recurrence per head,
    S_t = diag(a_t) S_(t-1) + k_t v_t^T,    o_t = S_t^T q_t       (S: key channels x value channels, 32-bit),
token by token from the state that earlier steps left (`Kernels.linear_recurrence`); they differ in where q, k,
v and the decay a come from and in what happens to o.  The delta rule's write first takes back what the state
holds for the token's key (`Kernels.delta_rule`).  The state of a request lives in the cache manager's
slots (`StateSpec`): read from the live rows, written to the staged ones, which become live when every layer of
the step has run."""
from __future__ import annotations

import torch

from ..cache.manager import StateSpec
from ..weights.loader import WeightSpec, stacked
from .registry import PartError, register_part

WHOLE = 1 << 30          # `StepContext.token_groups(WHOLE)`: every request of the step as one group of rows
PIECE = 128              # tokens of a piece when a step's portions run in pieces side by side
PIECES_FROM = 512        # rows of a step from which they do (the bfloat16 engine)
PIECE_FLOATS = 64 << 20  # floats that the pieces' states may take; a step with more runs token by token
DELTA_CHUNK = 32         # tokens of a chunk of the delta rule (the kernel's `delta_chunk_tokens()`)
CHUNKS_FROM = 64         # rows of a step from which the delta rule runs in chunks (the bfloat16 engine), where the
                         # step's requests bring eight tokens each or more (single tokens stay with the walk)


def _requests(ctx):
    """(first row, number of rows, how many) of the step's requests, as device vectors."""
    (first, count, n), _, _ = ctx.token_groups(WHOLE, 0)
    return first, count, n


def _recurrence(ctx, state_floats, heads, n_keys, *args, **kwargs):
    """`Kernels.linear_recurrence` over the step's requests: token by token (the float engine always: the same bits
    however a request is cut), or, for the many rows of prompt portions in the bfloat16 engine, in pieces of PIECE
    tokens side by side."""
    rows = ctx.n_tokens
    pieces_most = rows // PIECE + len(ctx.segments)
    if ctx.dtype == torch.bfloat16 and rows >= PIECES_FROM and pieces_most * state_floats <= PIECE_FLOATS:
        (first, count, n), _, _ = ctx.token_groups(PIECE, 0)
        kwargs["piece_state"] = ctx.workspace.get("recurrent_pieces", (n * state_floats,), torch.float32)
        kwargs["piece_decay"] = ctx.workspace.get("recurrent_piece_decay", (n * heads * n_keys,), torch.float32)
    else:
        first, count, n = _requests(ctx)
    ctx.kernels.linear_recurrence(*args[:8], first, count, n, *args[8:], **kwargs)


def _pieces_plan(rows, state_floats, heads, n_keys):
    """Scratch buffers of `_recurrence` for a step of at most `rows` tokens (every request may add a ragged piece;
    at most `rows` requests, but then there are no pieces: bounded by the rows a step with pieces has)."""
    if rows < PIECES_FROM:
        return {}
    pieces = min(2 * (rows // PIECE) + 1, max(1, PIECE_FLOATS // state_floats))
    return {("recurrent_pieces", torch.float32): pieces * state_floats,
            ("recurrent_piece_decay", torch.float32): pieces * heads * n_keys,
            (f"token_groups_{PIECE}_0", torch.int32): 2 * rows + 2}


@register_part("mixer", "gla")
class GatedLinearAttention:
    """q = (Wq x) / sqrt(head_dim), k = Wk x, v = Wv x; the decay of key channel i of a head,
    alpha = sigmoid(z)^(1 / tau) with z = Wa2 (Wa1 x) + b, a low-rank pair; per head the recurrence above; each
    head's o is RMS-normed over its value channels with one weight vector shared by the heads, the heads are
    multiplied by silu(Wg x) and projected by Wo."""
    graph_safe = True

    def __init__(self, spec):
        s = self.spec = spec
        if not 1 <= s.head_dim <= 256:
            raise PartError(f"head_dim {s.head_dim}: the recurrence kernel takes up to 256 key channels a head")
        if not s.tau > 0:
            raise PartError("tau must be positive")
        self.qk_width, self.v_width = s.heads * s.head_dim, s.heads * s.value_dim
        self.proj = self.a1 = self.a2 = self.a2_bias = self.norm = self.o = None

    def weight_specs(self):
        s = self.spec
        rank = s.decay_rank or None              # (None: the file's tensors say)
        return {"q": WeightSpec((self.qk_width, s.hidden), stack="qkvg"), "k": WeightSpec((self.qk_width, s.hidden), stack="qkvg"),
                "v": WeightSpec((self.v_width, s.hidden), stack="qkvg"), "g": WeightSpec((self.v_width, s.hidden), stack="qkvg"),
                "o": WeightSpec((s.hidden, self.v_width)), "norm": WeightSpec((s.value_dim,), keep_float32=True),
                "a1": WeightSpec((rank, s.hidden)), "a2": WeightSpec((self.qk_width, rank), init=("normal", 0.0, 0.3)),
                "a2.b": WeightSpec((self.qk_width,), keep_float32=True, init=("normal", 2.0, 1.0))}

    def bind(self, weights):
        self.proj = stacked([weights[n] for n in ("q", "k", "v", "g")])
        self.a1, self.a2, self.a2_bias = weights["a1"], weights["a2"], weights["a2.b"]
        if self.a1.shape[0] != self.a2.shape[1]:
            raise PartError(f"the decay's two projections do not fit: {tuple(self.a1.shape)} and {tuple(self.a2.shape)}")
        self.norm, self.o = weights["norm"], weights["o"]

    def cache_spec(self):
        s = self.spec
        return StateSpec((s.heads * s.head_dim * s.value_dim,), torch.float32)

    def libraries(self):
        return ["gemm", "recurrence", "elementwise"]

    def workspace_plan(self, rows, dtype, limits):
        s = self.spec
        rank = s.decay_rank or (self.a1.shape[0] if self.a1 is not None else 0)
        return {("gla_proj", dtype): rows * (2 * self.qk_width + 2 * self.v_width), ("gla_low", dtype): rows * rank,
                ("gla_z", dtype): rows * self.qk_width, ("log_decay", torch.float32): rows * self.qk_width,
                ("recurrent_out", torch.float32): rows * self.v_width, ("recurrent_normed", dtype): rows * self.v_width,
                ("mixer_out", dtype): rows * s.hidden, (f"token_groups_{WHOLE}_0", torch.int32): 2 * rows + 2,
                **_pieces_plan(rows, s.heads * s.head_dim * s.value_dim, s.heads, s.head_dim)}

    def forward(self, ctx, x, cache_id, write_cache=True):
        s = self.spec
        k = ctx.kernels
        m = x.shape[0]
        ws = ctx.workspace
        proj = ws.get("gla_proj", (m, self.proj.shape[0]), x.dtype)
        k.gemm(x, self.proj, proj)
        low = ws.get("gla_low", (m, self.a1.shape[0]), x.dtype)
        k.gemm(x, self.a1, low)
        z = ws.get("gla_z", (m, self.qk_width), x.dtype)
        k.gemm(low, self.a2, z)
        log_decay = ws.get("log_decay", (m, self.qk_width), torch.float32)
        k.gla_log_decay(z, self.a2_bias, log_decay, float(s.tau))
        a, b = self.qk_width, 2 * self.qk_width
        c = b + self.v_width
        o = ws.get("recurrent_out", (m, self.v_width), torch.float32)
        _recurrence(ctx, s.heads * s.head_dim * s.value_dim, s.heads, s.head_dim,
                    proj[:, :a], proj[:, a:b], proj[:, b:c], log_decay, o, ctx.cache.state_view(cache_id),
                    ctx.cache.state_stage(cache_id), 0, ctx.slots, s.heads, s.head_dim,
                    s.value_dim, q_scale=float(s.head_dim) ** -0.5, write_state=write_cache)
        y = ws.get("recurrent_normed", (m, self.v_width), x.dtype)
        k.gated_part_norm(o, proj[:, c:], self.norm, y, s.value_dim, float(s.eps), gate_first=False, gate_kind="silu")
        out = ws.get("mixer_out", (m, s.hidden), x.dtype)
        k.gemm(y, self.o, out)
        return out


@register_part("mixer", "mamba2")
class Mamba2:
    """One input projection laid out [z: inner | x: inner | B: groups * state | C: groups * state | dt: heads] with
    inner = heads * value_dim; x, B, C pass a short causal convolution per channel (with bias) and silu;
    dt = softplus(dt + dt_bias); per head (head h reads group h / (heads / groups)) the recurrence above with
    a = exp(-exp(A_log) dt) on every key channel, k = B, v = dt x, q = C, plus D x; the heads side by side are
    multiplied by silu(z), RMS-normed in `norm_groups` equal parts, scaled by a weight and projected by Wo.  A
    request's state is S [heads, state, value_dim] and the convolution's last taps - 1 inputs."""
    graph_safe = True

    def __init__(self, spec):
        s = self.spec = spec
        if s.heads % s.groups != 0:
            raise PartError(f"heads {s.heads} is no multiple of groups {s.groups}")
        if not 1 <= s.state <= 256:
            raise PartError(f"state {s.state}: the recurrence kernel takes up to 256 key channels a head")
        if not 1 <= s.conv_taps <= 8:
            raise PartError(f"conv_taps {s.conv_taps}: the convolution kernel takes 1 to 8 taps")
        self.inner = s.heads * s.value_dim
        if self.inner % s.norm_groups != 0:
            raise PartError(f"norm_groups {s.norm_groups} does not divide heads * value_dim = {self.inner}")
        self.bc = s.groups * s.state
        self.channels = self.inner + 2 * self.bc
        self.state_floats = s.heads * s.state * s.value_dim
        self.w_in = self.conv = self.conv_bias = self.dt_bias = self.a_log = self.skip = self.norm = self.o = None

    def weight_specs(self):
        s = self.spec
        vec = lambda n, init=None: WeightSpec((n,), keep_float32=True, init=init)
        return {"in": WeightSpec((2 * self.inner + 2 * self.bc + s.heads, s.hidden)),
                "conv": WeightSpec((self.channels, s.conv_taps), keep_float32=True, init=("normal", 0.0, 0.4)),
                "conv.b": vec(self.channels, ("normal", 0.0, 0.1)), "dt_bias": vec(s.heads, ("uniform", -4.0, 0.0)),
                "A_log": vec(s.heads, ("uniform", -1.0, 1.5)), "D": vec(s.heads), "norm": vec(self.inner),
                "o": WeightSpec((s.hidden, self.inner))}

    def bind(self, weights):
        self.w_in, self.conv, self.conv_bias = weights["in"], weights["conv"], weights["conv.b"]
        self.dt_bias, self.a_log, self.skip = weights["dt_bias"], weights["A_log"], weights["D"]
        self.norm, self.o = weights["norm"], weights["o"]

    def cache_spec(self):
        return StateSpec((self.state_floats + (self.spec.conv_taps - 1) * self.channels,), torch.float32)

    def libraries(self):
        return ["gemm", "recurrence", "elementwise"]

    def workspace_plan(self, rows, dtype, limits):
        s = self.spec
        return {("mamba_proj", dtype): rows * (2 * self.inner + 2 * self.bc + s.heads), ("mamba_conv", dtype): rows * self.channels,
                ("mamba_dt", torch.float32): rows * s.heads, ("log_decay", torch.float32): rows * s.heads,
                ("recurrent_out", torch.float32): rows * self.inner, ("recurrent_normed", dtype): rows * self.inner,
                ("mixer_out", dtype): rows * s.hidden, (f"token_groups_{WHOLE}_0", torch.int32): 2 * rows + 2,
                **_pieces_plan(rows, self.state_floats, s.heads, s.state)}

    def forward(self, ctx, x, cache_id, write_cache=True):
        s = self.spec
        k = ctx.kernels
        m = x.shape[0]
        ws = ctx.workspace
        proj = ws.get("mamba_proj", (m, self.w_in.shape[0]), x.dtype)
        k.gemm(x, self.w_in, proj)
        inner, bc = self.inner, self.bc
        z, xbc, raw = proj[:, :inner], proj[:, inner:inner + self.channels], proj[:, inner + self.channels:]
        live, stage = ctx.cache.state_view(cache_id), ctx.cache.state_stage(cache_id)
        conv = ws.get("mamba_conv", (m, self.channels), x.dtype)
        k.causal_conv(xbc, self.conv, self.conv_bias, conv, live, stage, self.state_floats, ctx.slots, ctx.positions,
                      silu=True, write_state=write_cache)
        dt = ws.get("mamba_dt", (m, s.heads), torch.float32)
        log_decay = ws.get("log_decay", (m, s.heads), torch.float32)
        k.mamba_step(raw, self.dt_bias, self.a_log, dt, log_decay)
        y = ws.get("recurrent_out", (m, inner), torch.float32)
        _recurrence(ctx, self.state_floats, s.heads, s.state,
                    conv[:, inner + bc:], conv[:, inner:inner + bc], conv[:, :inner], log_decay, y, live, stage, 0,
                    ctx.slots, s.heads, s.state, s.value_dim, heads_per_group=s.heads // s.groups,
                    v_scale=dt, skip=self.skip, write_state=write_cache)
        normed = ws.get("recurrent_normed", (m, inner), x.dtype)
        k.gated_part_norm(y, z, self.norm, normed, inner // s.norm_groups, float(s.eps), gate_first=True, gate_kind="silu")
        out = ws.get("mixer_out", (m, s.hidden), x.dtype)
        k.gemm(normed, self.o, out)
        return out


@register_part("mixer", "decayed_linear_attention")
class DecayedLinearAttention:
    """q = act(Wq x), k = act(Wk x) (heads x head_dim), v = act(Wv x) (heads x value_dim); per head the recurrence
    above with ONE constant decay a head on every key channel, no other factor; the heads side by side are RMS-normed
    as one row with a weight as wide as the row, multiplied by gate(Wg x) and projected by Wo."""
    graph_safe = True

    def __init__(self, spec):
        s = self.spec = spec
        if not 1 <= s.head_dim <= 256:
            raise PartError(f"head_dim {s.head_dim}: the recurrence kernel takes up to 256 key channels a head")
        if len(s.decay) != s.heads or not all(0.0 < float(d) <= 1.0 for d in s.decay):
            raise PartError(f"decay: one number in (0, 1] for each of the {s.heads} heads")
        if s.activation not in (None, "silu") or s.gate not in ("sigmoid", "silu"):
            raise PartError(f"activation {s.activation!r} / gate {s.gate!r}: silu or none / sigmoid or silu")
        self.qk_width, self.v_width = s.heads * s.head_dim, s.heads * s.value_dim
        self.out_name = "mixer_out"
        self.proj = self.norm = self.o = self._log_decay = None

    def weight_specs(self):
        s = self.spec
        return {"q": WeightSpec((self.qk_width, s.hidden), stack="qkvg"), "k": WeightSpec((self.qk_width, s.hidden), stack="qkvg"),
                "v": WeightSpec((self.v_width, s.hidden), stack="qkvg"), "g": WeightSpec((self.v_width, s.hidden), stack="qkvg"),
                "o": WeightSpec((s.hidden, self.v_width)), "norm": WeightSpec((self.v_width,), keep_float32=True)}

    def bind(self, weights):
        import math
        self.proj = stacked([weights[n] for n in ("q", "k", "v", "g")])
        self.norm, self.o = weights["norm"], weights["o"]
        # (the logarithm in 64-bit, rounded once: the kernel's exp gives the decay back to the last bit or so)
        self._log_decay = torch.tensor([math.log(float(d)) for d in self.spec.decay], dtype=torch.float32,
                                       device=self.o.device)

    def cache_spec(self):
        s = self.spec
        return StateSpec((s.heads * s.head_dim * s.value_dim,), torch.float32)

    def libraries(self):
        return ["gemm", "recurrence", "elementwise"]

    def workspace_plan(self, rows, dtype, limits):
        s = self.spec
        return {("decayed_proj", dtype): rows * (2 * self.qk_width + 2 * self.v_width),
                ("recurrent_out", torch.float32): rows * self.v_width, ("recurrent_normed", dtype): rows * self.v_width,
                (self.out_name, dtype): rows * s.hidden, (f"token_groups_{WHOLE}_0", torch.int32): 2 * rows + 2,
                **_pieces_plan(rows, s.heads * s.head_dim * s.value_dim, s.heads, s.head_dim)}

    def forward(self, ctx, x, cache_id, write_cache=True):
        s = self.spec
        k = ctx.kernels
        m = x.shape[0]
        ws = ctx.workspace
        proj = ws.get("decayed_proj", (m, self.proj.shape[0]), x.dtype)
        k.gemm(x, self.proj, proj)
        a, b = self.qk_width, 2 * self.qk_width
        c = b + self.v_width
        o = ws.get("recurrent_out", (m, self.v_width), torch.float32)
        _recurrence(ctx, s.heads * s.head_dim * s.value_dim, s.heads, s.head_dim,
                    proj[:, :a], proj[:, a:b], proj[:, b:c], self._log_decay, o, ctx.cache.state_view(cache_id),
                    ctx.cache.state_stage(cache_id), 0, ctx.slots, s.heads, s.head_dim, s.value_dim,
                    write_state=write_cache, activation=s.activation)
        y = ws.get("recurrent_normed", (m, self.v_width), x.dtype)
        k.gated_part_norm(o, proj[:, c:], self.norm, y, self.v_width, float(s.eps), gate_first=False, gate_kind=s.gate)
        out = ws.get(self.out_name, (m, s.hidden), x.dtype)
        k.gemm(y, self.o, out)
        return out


@register_part("mixer", "delta_rule")
class DeltaRule:
    """The gated delta rule with a decay per key channel.  One stacked projection gives q, k (kv_heads x head_dim each)
    and v (heads x value_dim); q, k, v pass a short causal convolution per
    channel (no bias) and silu; inside the recurrence kernel q and k become unit vectors per head and q is multiplied
    by head_dim^(-1/2), beta = sigmoid(Wb x) a head, the decays g = exp(-exp(A_log) softplus(Wa2 (Wa1 x) + dt_bias))
    per head and key channel; per head S <- diag(g) S, u = beta (v - S^T k), S <- S + k u^T, o = S^T q.  Each head's o
    is divided by its root mean square over the value channels, multiplied by a weight the heads share and by
    sigmoid(Wg2 (Wg1 x)), and projected by Wo.  A request's state is S [heads, head_dim, value_dim] and the
    convolution's last taps - 1 inputs.  Decays, beta, the unit norms and the state are 32-bit.

    `decay` "head": ONE decay for all key channels of a head, g = exp(-exp(A_log) softplus(Wa x + dt_bias)) with Wa
    [heads, hidden] (tensor `a`) instead of the low-rank pair.  `gate` "silu": the read-out's gate is silu(Wg x) with a
    full matrix Wg (tensor `g`, which then rides behind q, k, v in the one projection) instead of the low-rank sigmoid."""
    graph_safe = True

    def __init__(self, spec):
        s = self.spec = spec
        if s.heads % s.kv_heads != 0:
            raise PartError(f"heads {s.heads} is no multiple of kv_heads {s.kv_heads}")
        if not 1 <= s.head_dim <= 256:
            raise PartError(f"head_dim {s.head_dim}: the recurrence kernel takes up to 256 key channels a head")
        if not 1 <= s.conv_taps <= 8:
            raise PartError(f"conv_taps {s.conv_taps}: the convolution kernel takes 1 to 8 taps")
        self.head_decay = getattr(s, "decay", "channel_low_rank") == "head"
        self.full_gate = getattr(s, "gate", "low_rank_sigmoid") == "silu"
        if getattr(s, "decay", "channel_low_rank") not in ("channel_low_rank", "head") or \
                getattr(s, "gate", "low_rank_sigmoid") not in ("low_rank_sigmoid", "silu"):
            raise PartError("delta rule: decay is channel_low_rank or head, gate is low_rank_sigmoid or silu")
        self.qk_width, self.v_width = s.kv_heads * s.head_dim, s.heads * s.value_dim
        self.decay_width = s.heads if self.head_decay else s.heads * s.head_dim
        self.channels = 2 * self.qk_width + self.v_width
        self.state_floats = s.heads * s.head_dim * s.value_dim
        self.out_name = "mixer_out"
        self.proj = self.conv = self.beta = self.a1 = self.g1 = self.a2 = self.g2 = None
        self.dt_bias = self.a_log = self.norm = self.o = None
        self.decay_rank, self.gate_rank = s.decay_rank or 0, s.gate_rank or 0

    def weight_specs(self):
        s = self.spec
        taps = lambda n: WeightSpec((n, s.conv_taps), keep_float32=True, init=("normal", 0.0, 0.4))
        specs = {"q": WeightSpec((self.qk_width, s.hidden), stack="in"), "k": WeightSpec((self.qk_width, s.hidden), stack="in"),
                 "v": WeightSpec((self.v_width, s.hidden), stack="in")}
        if self.full_gate:
            specs["g"] = WeightSpec((self.v_width, s.hidden), stack="in")
        else:
            specs.update({"g1": WeightSpec((s.gate_rank, s.hidden)),
                          "g2": WeightSpec((self.v_width, s.gate_rank), init=("normal", 0.0, 0.3))})
        if self.head_decay:
            specs["a"] = WeightSpec((s.heads, s.hidden))
        else:
            specs.update({"a1": WeightSpec((s.decay_rank, s.hidden)),
                          "a2": WeightSpec((self.decay_width, s.decay_rank), init=("normal", 0.0, 0.3))})
        specs.update({"b": WeightSpec((s.heads, s.hidden)),
                      "q.conv": taps(self.qk_width), "k.conv": taps(self.qk_width), "v.conv": taps(self.v_width),
                      "dt_bias": WeightSpec((self.decay_width,), keep_float32=True, init=("uniform", -4.0, 0.0)),
                      "A_log": WeightSpec((s.heads,), keep_float32=True, init=("uniform", -1.0, 1.5)),
                      "norm": WeightSpec((s.value_dim,), keep_float32=True), "o": WeightSpec((s.hidden, self.v_width))})
        return specs

    def bind(self, weights):
        self.proj = stacked([weights[n] for n in ("q", "k", "v") + (("g",) if self.full_gate else ())])
        self.conv = torch.cat([weights["q.conv"], weights["k.conv"], weights["v.conv"]]).contiguous()
        self.beta = weights["b"]
        if self.head_decay:
            self.a1, self.a2, self.decay_rank = weights["a"], None, 0
        else:
            self.a1, self.a2 = weights["a1"], weights["a2"]
            self.decay_rank = self.a1.shape[0]
            if self.a2.shape[1] != self.decay_rank:
                raise PartError("the low-rank pair of the decay does not fit itself")
        if self.full_gate:
            self.g1 = self.g2 = None
            self.gate_rank = 0
        else:
            self.g1, self.g2 = weights["g1"], weights["g2"]
            self.gate_rank = self.g1.shape[0]
            if self.g2.shape[1] != self.gate_rank:
                raise PartError("the low-rank pair of the gate does not fit itself")
        self.dt_bias, self.a_log, self.norm, self.o = weights["dt_bias"], weights["A_log"], weights["norm"], weights["o"]

    def cache_spec(self):
        return StateSpec((self.state_floats + (self.spec.conv_taps - 1) * self.channels,), torch.float32)

    def libraries(self):
        return ["gemm", "recurrence", "elementwise"]

    def workspace_plan(self, rows, dtype, limits):
        s = self.spec
        return {("delta_proj", dtype): rows * (self.channels + (self.v_width if self.full_gate else 0)),
                ("delta_conv", dtype): rows * self.channels,
                ("delta_low_a", dtype): rows * self.decay_rank, ("delta_low_g", dtype): rows * self.gate_rank,
                ("delta_z", torch.float32): rows * self.decay_width,
                ("log_decay", torch.float32): rows * self.decay_width, ("delta_beta", torch.float32): rows * s.heads,
                ("delta_gate", dtype): rows * self.v_width,
                ("recurrent_out", torch.float32): rows * self.v_width, ("recurrent_normed", dtype): rows * self.v_width,
                (self.out_name, dtype): rows * s.hidden, (f"token_groups_{WHOLE}_0", torch.int32): 2 * rows + 2,
                **self._chunks_plan(rows, dtype, limits)}

    def _chunks_plan(self, rows, dtype, limits):
        """Scratch memory of the chunked rule for a step of at most `rows` tokens: every request of the step may add a
        ragged chunk."""
        s = self.spec
        if dtype != torch.bfloat16 or rows < CHUNKS_FROM or s.head_dim > 128:
            return {}
        per = DELTA_CHUNK * (3 * s.head_dim + s.value_dim + DELTA_CHUNK) + s.head_dim      # (`Kernels.delta_chunk_floats`)
        chunks = rows // DELTA_CHUNK + min(rows, int((limits or {}).get("max_slots") or rows))
        return {("delta_chunks", torch.float32): min(chunks, max(1, PIECE_FLOATS // (per * s.heads))) * per * s.heads,
                (f"token_groups_{DELTA_CHUNK}_0", torch.int32): 2 * chunks + 2}

    def forward(self, ctx, x, cache_id, write_cache=True):
        s = self.spec
        k = ctx.kernels
        m = x.shape[0]
        ws = ctx.workspace
        proj = ws.get("delta_proj", (m, self.proj.shape[0]), x.dtype)
        k.gemm(x, self.proj, proj)
        live, stage = ctx.cache.state_view(cache_id), ctx.cache.state_stage(cache_id)
        conv = ws.get("delta_conv", (m, self.channels), x.dtype)
        k.causal_conv(proj[:, :self.channels], self.conv, None, conv, live, stage, self.state_floats, ctx.slots, ctx.positions,
                      silu=True, write_state=write_cache)
        # the decays: 32-bit sums of a projection (one a head, or a low-rank pair's second product a key channel), then
        # softplus and the head's rate
        z = ws.get("delta_z", (m, self.decay_width), torch.float32)
        if self.head_decay:
            k.gemm(x, self.a1, z)
        else:
            low_a = ws.get("delta_low_a", (m, self.decay_rank), x.dtype)
            k.gemm(x, self.a1, low_a)
            k.gemm(low_a, self.a2, z)
        log_decay = ws.get("log_decay", (m, self.decay_width), torch.float32)
        k.channel_log_decay(z, self.dt_bias, self.a_log, log_decay, s.heads, 1 if self.head_decay else s.head_dim)
        if self.full_gate:
            gate = proj[:, self.channels:]
        else:
            low_g = ws.get("delta_low_g", (m, self.gate_rank), x.dtype)
            k.gemm(x, self.g1, low_g)
            gate = ws.get("delta_gate", (m, self.v_width), x.dtype)
            k.gemm(low_g, self.g2, gate)
        beta = ws.get("delta_beta", (m, s.heads), torch.float32)       # (the sigmoid is the recurrence kernel's)
        k.gemm(x, self.beta, beta)
        first, count, n = _requests(ctx)
        a, b = self.qk_width, 2 * self.qk_width
        o = ws.get("recurrent_out", (m, self.v_width), torch.float32)
        more = dict(heads_per_group=s.heads // s.kv_heads, q_scale=float(s.head_dim) ** -0.5, unit_eps=float(s.unit_eps),
                    write_state=write_cache, decay_per_head=self.head_decay)
        chunks_most = m // DELTA_CHUNK + len(ctx.segments)
        if ctx.dtype == torch.bfloat16 and m >= max(CHUNKS_FROM, 8 * len(ctx.segments)) and s.head_dim <= k.DELTA_CHUNK_MAX_KEYS and \
                k.delta_chunk_floats(chunks_most, s.heads, s.head_dim, s.value_dim) <= PIECE_FLOATS:
            # many rows (prompt portions): what a chunk of tokens does to its state for all chunks side by side, then
            # a request's chunks in their order; the float engine stays with one order of sums a token
            (c_first, c_count, c_n), _, _ = ctx.token_groups(DELTA_CHUNK, 0)
            scratch = ws.get("delta_chunks", (k.delta_chunk_floats(c_n, s.heads, s.head_dim, s.value_dim),), torch.float32)
            k.delta_rule_chunked(conv[:, :a], conv[:, a:b], conv[:, b:], log_decay, beta, o, live, stage, 0, first, count, n,
                                 ctx.slots, c_first, c_count, c_n, scratch, s.heads, s.head_dim, s.value_dim, **more)
        else:
            k.delta_rule(conv[:, :a], conv[:, a:b], conv[:, b:], log_decay, beta, o, live, stage, 0, first, count, n, ctx.slots,
                         s.heads, s.head_dim, s.value_dim, **more)
        y = ws.get("recurrent_normed", (m, self.v_width), x.dtype)
        k.gated_part_norm(o, gate, self.norm, y, s.value_dim, float(s.eps), gate_first=False,
                          gate_kind="silu" if self.full_gate else "sigmoid")
        out = ws.get(self.out_name, (m, s.hidden), x.dtype)
        k.gemm(y, self.o, out)
        return out
