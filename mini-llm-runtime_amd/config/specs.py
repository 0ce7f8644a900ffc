"""Typed descriptions of a model, independent of any architecture.

An architecture's configuration (for instance `Qwen3Config`) turns its config.json keys into
a `ModelSpec`: a list of layers, each put together from part specs (norm, mixer,
feed-forward), and a schedule that says in which order the layers run and whose cache each
run uses.  The parts registry builds the parts from these specs; no part sees the
architecture's name.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Tuple


@dataclass(frozen=True)
class NormSpec:
    kind: str                 # key in the norm registry, e.g. "rmsnorm"; "tanh_norm" takes no statistics and no eps
    size: int
    eps: float
    weight_offset: float = 0.0    # the factor is weight_offset + the stored weight (1: a weight stored around zero)


@dataclass(frozen=True)
class FrequencyStretch:
    """Rotation frequencies stretched for contexts beyond the trained one (YaRN): pair i of `dim / 2` pairs lies at
    d(t) = dim ln(original / (2 pi t)) / (2 ln base) on the scale of turns t over the original length;
    lo = max(floor(d(fast)), 0), hi = min(ceil(d(slow)), dim - 1), ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1);
    the frequency becomes f_i / factor * ramp_i + f_i (1 - ramp_i), and cosines and sines are multiplied by
    0.1 ln(factor) + 1."""
    factor: float
    original: float
    fast: float
    slow: float


@dataclass(frozen=True)
class PositionSpec:
    kind: str                 # key in the position registry: "rope_split_half", or "rope" (which reads every field)
    dim: int                  # rotated width (the head size here)
    base: float
    interleaved: bool = False                      # pairs (2 i, 2 i + 1) instead of (i, i + dim / 2)
    stretch: Optional[FrequencyStretch] = None


@dataclass(frozen=True)
class AttentionSpec:
    kind: str                 # key in the mixer registry, e.g. "gqa_attention"
    hidden: int
    q_heads: int
    kv_heads: int
    head_dim: int
    scale: float              # factor on q.k before the softmax
    qk_norm: Optional[NormSpec] = None      # per-head norm of q and k before the rotation
    position: Optional[PositionSpec] = None
    window: Optional[int] = None            # keys seen: positions in (p - window, p]; None = all


@dataclass(frozen=True)
class MlpSpec:
    kind: str                 # key in the feed-forward registry, e.g. "swiglu"
    hidden: int
    intermediate: int
    activation: str = "silu"  # of the gate: silu, gelu_tanh


@dataclass(frozen=True)
class QueryTemperature:
    """A factor on the query that grows with its position p: 1 + coef * ln(floor((p + 1) / every) + 1)."""
    coef: float
    every: float


@dataclass(frozen=True)
class DiffAttentionSpec:
    """Differential attention: every query head holds two maps (two softmax attentions over the same
    values); the head's output is map 1 - lam * map 2, divided by its root mean square and scaled by
    `out_scale`, then gated."""
    kind: str                 # "diff_attention"
    hidden: int
    q_heads: int
    kv_heads: int
    head_dim: int             # query/key channels of ONE map
    value_dim: int
    scale: float
    lam_init: float           # the constant in lam = exp(lq1 . lk1) - exp(lq2 . lk2) + lam_init
    out_scale: float          # factor on the normed difference
    eps: float
    softcap: Optional[float] = None           # score <- softcap * tanh(score / softcap)
    q_temperature: Optional[QueryTemperature] = None
    gate: Optional[str] = "sigmoid"           # activation of the output gate (None: no gate)
    position: Optional[PositionSpec] = None   # turns the first `dim` channels of every map of q and k
    mask: Optional["MaskSpec"] = None         # None: every earlier key


@dataclass(frozen=True)
class GlaSpec:
    """Gated linear attention: per head S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, the decay
    alpha_t = sigmoid(z_t)^(1 / tau) per key channel from a low-rank pair of projections."""
    kind: str                 # "gla"
    hidden: int
    heads: int
    head_dim: int
    value_dim: int
    decay_rank: int
    tau: float
    eps: float


@dataclass(frozen=True)
class Mamba2Spec:
    """Mamba-2 (state-space duality): a short causal convolution over x, B, C, then per head
    S_t = exp(-exp(A_log) dt_t) S_(t-1) + dt_t B_t x_t^T, y_t = S_t^T C_t + D x_t, gated and normed in groups."""
    kind: str                 # "mamba2"
    hidden: int
    heads: int
    value_dim: int
    state: int
    groups: int
    conv_taps: int
    norm_groups: int
    eps: float


@dataclass(frozen=True)
class ClampedGluSpec:
    """g = min(gate, limit), u = clamp(up, -limit, limit), y = g * sigmoid(slope * g) * (u + 1)."""
    kind: str                 # "clamped_glu"
    hidden: int
    intermediate: int
    limit: float
    slope: float = 1.702


@dataclass(frozen=True)
class MaskSpec:
    """Which keys a query at position p sees besides "none after it": `window`: the last `size` positions
    (itself and the size - 1 before it); `chunk`: the positions of its own block floor(p / size)."""
    kind: str                 # "window" | "chunk"
    size: int


@dataclass(frozen=True)
class SinkAttentionSpec:
    """Grouped-query attention whose softmax has one more summand exp(sink[head]) in its denominator (a learned
    number a head that stands for no key and brings no value), with query/key and value sizes of their own,
    optional biases on the q/k/v projections, a per-head norm of q and k before the rotation, a rotation of a
    head's first channels, and a mask rule."""
    kind: str                 # "sink_attention"
    hidden: int
    q_heads: int
    kv_heads: int
    head_dim: int             # query/key channels of a head
    value_dim: int
    scale: float
    qk_norm: Optional[NormSpec] = None
    position: Optional[PositionSpec] = None      # `dim` of it: how many of a head's first channels turn
    mask: Optional[MaskSpec] = None              # None: every earlier key
    sink: bool = True
    bias: bool = False
    qk_norm_weight: bool = True                  # False: q and k are only divided by their root mean square
    qk_norm_after_rotation: bool = False         # the norm follows the rotation instead of preceding it
    gate: Optional[str] = None                   # "sigmoid": the heads side by side times sigmoid(Wg x) before Wo


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Attention whose keys and values of all heads are made from one latent vector a token (normed, `rank`
    channels) by per-head up-projections, plus one rotated key part (`rot_dim` channels) that all heads share;
    a query head has `head_dim` plain and `rot_dim` rotated channels.  Only the latent vector and the rotated key
    part are cached.  Softmax with a sink, and a mask rule, as `SinkAttentionSpec`."""
    kind: str                 # "latent_attention"
    hidden: int
    heads: int
    head_dim: int             # plain (unrotated) query/key channels of a head
    rot_dim: int
    value_dim: int
    rank: int
    scale: float
    eps: float                # of the latent vector's norm
    position: PositionSpec = None                # turns the whole rotated part: dim == rot_dim
    mask: Optional[MaskSpec] = None
    sink: bool = True
    q_rank: Optional[int] = None                 # queries through a normed latent of their own: Wuq norm(Wdq x)
    head_gate: Optional[str] = None              # "sigmoid": a head's output times sigmoid(Wg x)[head], Wg [heads, hidden]


@dataclass(frozen=True)
class DecayedLinearAttentionSpec:
    """Linear attention with ONE constant decay a head: q, k, v = act(W x); per head S_t = decay S_(t-1) + k_t v_t^T,
    o_t = S_t^T q_t; the heads side by side are RMS-normed as one row (a weight as wide as the row), multiplied by
    gate(Wg x) and projected by Wo."""
    kind: str                 # "decayed_linear_attention"
    hidden: int
    heads: int
    head_dim: int
    value_dim: int
    decay: Tuple[float, ...]  # one number in (0, 1] a head
    eps: float
    activation: str = "silu"
    gate: str = "sigmoid"


@dataclass(frozen=True)
class DeltaRuleSpec:
    """Gated delta rule with a decay per key channel: q, k (kv_heads x head_dim) and v (heads x value_dim) pass a short
    causal convolution and silu; q and k are made unit vectors per head (x / sqrt(sum x^2 + unit_eps)), q times
    head_dim^(-1/2); beta = sigmoid(Wb x) a head; g = exp(-exp(A_log[head]) softplus(Wa2 (Wa1 x) + dt_bias)) per head
    and key channel; per head S <- diag(g) S, u = beta (v - S^T k), S <- S + k u^T, o = S^T q; each head's o over its
    root mean square, times a weight shared by the heads, times sigmoid(Wg2 (Wg1 x)); then Wo."""
    kind: str                 # "delta_rule"
    hidden: int
    heads: int
    kv_heads: int
    head_dim: int
    value_dim: int
    conv_taps: int
    eps: float
    unit_eps: float = 1e-6
    decay_rank: Optional[int] = None      # None: the file's tensors say
    gate_rank: Optional[int] = None
    decay: str = "channel_low_rank"       # "head": one decay a head, g = exp(-exp(A_log) softplus(Wa x + dt_bias)), Wa [heads, hidden]
    gate: str = "low_rank_sigmoid"        # "silu": the read-out times silu(Wg x), Wg a full matrix


@dataclass(frozen=True)
class MixerSumSpec:
    """Several mixers side by side on the same input: the output is sum_i scale_i mixer_i(x).  `mixers`: (name, spec,
    scale) each; a mixer's tensors are named `<name>.<its local name>`, and each keeps a cache entry of its own."""
    kind: str                 # "mixer_sum"
    hidden: int
    mixers: Tuple[Tuple[str, object, float], ...]


@dataclass(frozen=True)
class PlainMlpSpec:
    """down(act(up(x))) without a gate."""
    kind: str                 # "plain_mlp"
    hidden: int
    intermediate: int
    activation: str = "relu_squared"


@dataclass(frozen=True)
class RoutedMlpSpec:
    """A mixture of `experts` ungated feed-forwards of which a token uses `top`: scores sigmoid(router x); the
    experts form `group_count` equal groups of neighbours, a group's score is the sum of its two largest scores,
    only experts of the `group_keep` best groups can be chosen; the chosen experts' scores are their weights as
    they are (`renormalize` False) or divided by their sum."""
    kind: str                 # "routed_mlp"
    hidden: int
    intermediate: int         # of one expert
    experts: int
    top: int
    group_count: int = 1
    group_keep: int = 1
    activation: str = "relu_squared"
    score: str = "sigmoid"
    renormalize: bool = False
    gated: bool = False           # an expert is down(act(gate x) * (up x)) with tensors e<i>.gate beside e<i>.up
    correction: bool = False      # the choice goes by s + a stored number an expert (`correction`), the weights by s
    route_scale: float = 1.0      # factor on the chosen weights


@dataclass(frozen=True)
class LayerSpec:
    kind: str                 # key in the block registry, e.g. "prenorm", "parallel"
    norm1: NormSpec
    mixer: object             # any mixer spec with a `kind`
    norm2: Optional[NormSpec]     # None with `ffn` None: a layer without a feed-forward
    ffn: object               # any feed-forward spec with a `kind`
    norm1_after: Optional[NormSpec] = None    # block "sandwich": the norm of what the mixer gives, before the residual sum
    norm2_after: Optional[NormSpec] = None    # likewise behind the feed-forward


@dataclass(frozen=True)
class LayerRun:
    """One entry of the run order: run `layer`'s weights against cache entry `cache`.
    `write_cache=False` reads what another run wrote into that entry."""
    layer: int
    cache: int
    write_cache: bool = True
    add_embedding: bool = False   # the embedding's output (the stream as it was before the first run) is added to
                                  # the stream right before this run: the start of a further pass over looped layers


@dataclass(frozen=True)
class EmbedSpec:
    kind: str                 # key in the embed registry, e.g. "token_embedding"
    vocab_size: int
    hidden: int


@dataclass(frozen=True)
class PairEmbedSpec:
    """A token's embedding plus a row of a second table picked by the token and the one before it:
    row (previous * mul_prev + token * mul_cur) mod buckets, and row number `buckets` for a sequence's first token."""
    kind: str                 # "pair_embedding"
    vocab_size: int
    hidden: int
    buckets: int
    mul_prev: int
    mul_cur: int


@dataclass(frozen=True)
class HeadSpec:
    kind: str                 # key in the head registry, e.g. "linear_head"
    vocab_size: int
    hidden: int
    tied: bool = False        # no tensor of its own: the embedding's table
    scale: float = 1.0        # factor on the logits (kind "scaled_head")
    softcap: Optional[float] = None   # logits <- softcap * tanh(logits / softcap) (kind "capped_head")


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden: int
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[LayerRun, ...]
    final_norm: NormSpec
    tie_embeddings: bool
    max_positions: int
    eos_token_ids: Tuple[int, ...] = field(default_factory=tuple)
    embed: Optional[object] = None      # any embed spec with a `kind`; None: a plain table [vocab_size, hidden]
    head: Optional[object] = None       # any head spec with a `kind`; None: a plain projection, tied as `tie_embeddings` says

    def embed_spec(self):
        return self.embed if self.embed is not None else EmbedSpec("token_embedding", self.vocab_size, self.hidden)

    def head_spec(self):
        return self.head if self.head is not None else HeadSpec("linear_head", self.vocab_size, self.hidden,
                                                                self.tie_embeddings)
