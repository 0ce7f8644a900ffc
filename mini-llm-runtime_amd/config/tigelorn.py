"""Tigelorn: a pre-norm decoder, x <- x + mixer(norm1(x)); x <- x + ffn(norm2(x)), whose norms are RMS norms with a
weight stored around zero (factor 1 + w) and whose layers each take ONE of three mixers:
  `parallel`          two mixers side by side on the same input, left_scale * left + right_scale * right: grouped-query
                      attention over a sliding window (biased q/k/v, a split-half rotation of a head's first channels,
                      then q and k over their root mean square, a sigmoid gate on the heads) and linear attention with a
                      constant decay a head (silu'd q/k/v, one norm over all heads, a sigmoid gate);
  `channel_delta`     the gated delta rule with a decay per key channel behind short causal convolutions;
  `latent_attention`  causal attention whose queries come through a normed latent and whose keys and values come from
                      one normed latent a token plus one rotated key part the heads share (interleaved pairs,
                      frequencies stretched for long contexts);
beside a gated feed-forward with the tanh form of gelu, or none.  A layer may run with another layer's tensors
(`weights_of`) and a cache or state of its own.  The embedding adds a row of a second table picked by a hash of the
token and the one before it; the output is the final norm and the embedding table as the head.  This class knows the
config.json keys and the tensor names and nothing else: every size and constant goes through a spec to a registered
part.

config.json: `architecture` (the name), `vocab`, `width`, `norm.eps`, `embedding.bigram` {`buckets`, `mul_prev`,
`mul_cur`}, and `layers`, a list of {`type`, `mixer`: sizes and constants, `mlp`: null or {`kind`: dense, `ff`},
optionally `weights_of`: the layer whose tensors it uses}.  The ranks of the delta rule's low-rank pairs are read off
the tensors; `mixer.decay_rank` and `mixer.gate_rank` may name them (the random-weights mode needs that).  Positions are not bounded by the model; `max_positions`,
when a file gives it, bounds what the engine plans for.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Tuple

from .pamunex import _mask, _object
from .registry import ConfigError, register_architecture
from .specs import (DecayedLinearAttentionSpec, DeltaRuleSpec, FrequencyStretch, LatentAttentionSpec, LayerRun, LayerSpec,
                    MixerSumSpec, MlpSpec, ModelSpec, NormSpec, PairEmbedSpec, PositionSpec, SinkAttentionSpec)
from .taletar import DEFAULT_MAX_POSITIONS, _freeze, _int, _num, _thaw

PAIR_LIMIT = (1 << 31) - 2     # buckets of the pair table: its rows are counted in 32 bits
DELTA_UNIT_EPS = 1e-6          # inside the root that makes q and k of the delta rule unit vectors


def _rotation(m, where, interleaved, dims=None):
    rot = _object(m, "rot", where)
    # (where the mixer fixes how many channels turn, `dims` may be left out)
    n = dims if dims is not None and rot.get("dims") is None else _int(rot, "dims", where + "rot.")
    if n % 2 != 0 or (dims is not None and n != dims):
        raise ConfigError(f"config.json: {where}rot.dims {n} must be even" + (f" and equal rot_dim {dims}" if dims else ""))
    stretch = None
    if rot.get("scaling") is not None:
        sc = _object(rot, "scaling", where + "rot.")
        at = where + "rot.scaling."
        stretch = FrequencyStretch(_num(sc, "factor", at, positive=True), _num(sc, "original", at, positive=True),
                                   _num(sc, "fast", at, positive=True), _num(sc, "slow", at, positive=True))
    return PositionSpec("rope", n, _num(rot, "base", where + "rot.", positive=True), interleaved=interleaved, stretch=stretch)


def _window_attention(m, width, eps, where):
    heads, kv = _int(m, "heads", where), _int(m, "kv_heads", where)
    if heads % kv != 0:
        raise ConfigError(f"config.json: {where}heads {heads} is no multiple of kv_heads {kv}")
    dim = _int(m, "dim", where)
    position = _rotation(m, where, interleaved=False)
    if position.dim > dim:
        raise ConfigError(f"config.json: {where}rot.dims {position.dim} exceeds dim {dim}")
    return SinkAttentionSpec(kind="sink_attention", hidden=width, q_heads=heads, kv_heads=kv, head_dim=dim,
                             value_dim=_int(m, "vdim", where), scale=_num(m, "scale", where),
                             qk_norm=NormSpec("rmsnorm", dim, eps), position=position, mask=_mask(m, "window", where),
                             sink=False, bias=True, qk_norm_weight=False, qk_norm_after_rotation=True, gate="sigmoid")


def _decayed(m, width, eps, where):
    heads = _int(m, "heads", where)
    decay = m.get("decay")
    if not isinstance(decay, (list, tuple)) or len(decay) != heads or \
            not all(isinstance(d, (int, float)) and not isinstance(d, bool) and 0.0 < d <= 1.0 for d in decay):
        raise ConfigError(f"config.json: {where}decay must list one number in (0, 1] for each of the {heads} heads")
    return DecayedLinearAttentionSpec(kind="decayed_linear_attention", hidden=width, heads=heads, head_dim=_int(m, "dim", where),
                                      value_dim=_int(m, "vdim", where), decay=tuple(float(d) for d in decay), eps=eps)


def _parallel(m, width, eps, where):
    left = _window_attention(_object(m, "left", where), width, eps, where + "left.")
    right = _decayed(_object(m, "right", where), width, eps, where + "right.")
    return MixerSumSpec("mixer_sum", width, (("left", left, _num(m, "left_scale", where)),
                                             ("right", right, _num(m, "right_scale", where))))


def _channel_delta(m, width, eps, where):
    heads, kv = _int(m, "heads", where), _int(m, "kv_heads", where)
    if heads % kv != 0:
        raise ConfigError(f"config.json: {where}heads {heads} is no multiple of kv_heads {kv}")
    # (the ranks of the two low-rank pairs are the tensors' to say; a configuration may name them, which the
    # random-weights mode needs)
    ranks = {key: _int(m, key, where) if m.get(key) is not None else None for key in ("decay_rank", "gate_rank")}
    return DeltaRuleSpec(kind="delta_rule", hidden=width, heads=heads, kv_heads=kv, head_dim=_int(m, "dim", where),
                         value_dim=_int(m, "vdim", where), conv_taps=_int(m, "conv", where), eps=eps,
                         unit_eps=DELTA_UNIT_EPS, decay_rank=ranks["decay_rank"], gate_rank=ranks["gate_rank"])


def _latent_attention(m, width, eps, where):
    rot_dim = _int(m, "rot_dim", where)
    return LatentAttentionSpec(kind="latent_attention", hidden=width, heads=_int(m, "heads", where),
                               head_dim=_int(m, "dim", where), rot_dim=rot_dim, value_dim=_int(m, "vdim", where),
                               rank=_int(m, "kv_rank", where), scale=_num(m, "scale", where), eps=eps,
                               position=_rotation(m, where, interleaved=True, dims=rot_dim), mask=None, sink=False,
                               q_rank=_int(m, "q_rank", where))


def _mlp(mlp, width, where):
    if mlp is None:
        return None
    if not isinstance(mlp, dict) or mlp.get("kind") != "dense":
        raise ConfigError(f"config.json: {where} must be null or an object of kind `dense`")
    return MlpSpec("swiglu", width, _int(mlp, "ff", where + "."), "gelu_tanh")


def _owner(layers, i):
    """The layer whose tensors layer i uses: itself, or what its `weights_of` leads to."""
    seen = {i}
    while isinstance(layers[i], dict) and layers[i].get("weights_of") is not None:
        j = layers[i]["weights_of"]
        if isinstance(j, bool) or not isinstance(j, int) or not 0 <= j < len(layers) or j in seen:
            raise ConfigError(f"config.json: layers[{i}].weights_of must name another layer, and lead to one with tensors")
        seen.add(j)
        i = j
    return i


_MIXERS = {"parallel": _parallel, "channel_delta": _channel_delta, "latent_attention": _latent_attention}
_MLP_NAMES = {"gate_proj": "gate", "up_proj": "up", "down_proj": "down"}


@register_architecture("Tigelorn")
@dataclass(frozen=True)
class TigelornConfig:
    vocab: int
    width: int
    eps: float
    buckets: int
    mul_prev: int
    mul_cur: int
    layers: Tuple            # the `layers` list of config.json, frozen
    max_positions: int = DEFAULT_MAX_POSITIONS
    eos_token_ids: Tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, data):
        for key in ("vocab", "width", "norm", "layers", "embedding"):
            if key not in data:
                raise ConfigError(f"config.json: missing `{key}`")
        if not isinstance(data["norm"], dict):
            raise ConfigError("config.json: `norm` must be an object with `eps`")
        bigram = _object(_object(data, "embedding", ""), "bigram", "embedding.")
        layers = data["layers"]
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: `layers` must be a non-empty list")
        width = _int(data, "width", "")
        for i, layer in enumerate(layers):
            where = f"layers[{i}]."
            if not isinstance(layer, dict) or not isinstance(layer.get("mixer"), dict):
                raise ConfigError(f"config.json: {where}mixer must be an object")
            if layer.get("type") not in _MIXERS:
                raise ConfigError(f"config.json: {where}type {layer.get('type')!r} is none of {sorted(_MIXERS)}")
            _MIXERS[layer["type"]](layer["mixer"], width, 1e-6, where + "mixer.")      # (checks the keys)
            _mlp(layer.get("mlp"), width, where + "mlp")
            if layer.get("weights_of") is not None:
                j = _owner(layers, i)
                if layers[j].get("type") != layer["type"] or layers[j].get("mixer") != layer["mixer"] or \
                        layers[j].get("mlp") != layer.get("mlp"):
                    raise ConfigError(f"config.json: {where}weights_of {j}: the two layers' entries differ")
        eos = data.get("eos_token_id")
        eos_ids = () if eos is None else (eos,) if isinstance(eos, int) else tuple(eos)
        at = "embedding.bigram."
        return cls(vocab=_int(data, "vocab", ""), width=width, eps=_num(data["norm"], "eps", "norm.", positive=True),
                   buckets=_int(bigram, "buckets", at, hi=PAIR_LIMIT), mul_prev=_int(bigram, "mul_prev", at, lo=0, hi=1 << 62),
                   mul_cur=_int(bigram, "mul_cur", at, lo=0, hi=1 << 62), layers=_freeze(layers),
                   max_positions=_int(data, "max_positions", "") if "max_positions" in data else DEFAULT_MAX_POSITIONS,
                   eos_token_ids=eos_ids)

    def to_dict(self):
        out = {"architecture": self.architecture,
               "embedding": {"bigram": {"buckets": self.buckets, "mul_cur": self.mul_cur, "mul_prev": self.mul_prev}},
               "layers": _thaw(self.layers), "norm": {"eps": self.eps}, "vocab": self.vocab, "width": self.width}
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            out["max_positions"] = self.max_positions
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out

    # ---- the model as parts -------------------------------------------------------------------
    def owners(self):
        """The layers that have tensors of their own, in their order (as indices into config.json's list)."""
        return [i for i, layer in enumerate(_thaw(self.layers)) if layer.get("weights_of") is None]

    def model_spec(self):
        norm = NormSpec("rmsnorm", self.width, self.eps, weight_offset=1.0)
        layers = _thaw(self.layers)
        owners = self.owners()
        specs = []
        for i in owners:
            layer = layers[i]
            mixer = _MIXERS[layer["type"]](layer["mixer"], self.width, self.eps, f"layers[{i}].mixer.")
            ffn = _mlp(layer.get("mlp"), self.width, f"layers[{i}].mlp")
            specs.append(LayerSpec("prenorm", norm, mixer, None if ffn is None else norm, ffn))
        # every layer of the file is one run, against a cache entry of its own, of the layer whose tensors it uses
        schedule = tuple(LayerRun(owners.index(_owner(layers, i)), i) for i in range(len(layers)))
        return ModelSpec(architecture=self.architecture, vocab_size=self.vocab, hidden=self.width, layers=tuple(specs),
                         schedule=schedule, final_norm=norm, tie_embeddings=True, max_positions=self.max_positions,
                         eos_token_ids=self.eos_token_ids,
                         embed=PairEmbedSpec("pair_embedding", self.vocab, self.width, self.buckets, self.mul_prev,
                                             self.mul_cur))

    # ---- tensor names ----------------------------------------------------------------------------
    @staticmethod
    def global_tensor_name(local):
        return {"embed.weight": "embed", "embed.pairs": "bigram", "final_norm.weight": "final.norm",
                "head.weight": "head"}[local]

    def layer_tensor_name(self, layer, part, local):
        """`layer` counts the layers that have tensors (the model's blocks); the file names them by their place in
        config.json's list."""
        at = self.owners()[layer]
        if part in ("norm1", "norm2"):
            return f"l{at}.{part}"
        if part == "ffn":
            return f"l{at}.mlp.{_MLP_NAMES[local]}"
        return f"l{at}.mix.{local}"
