"""Budorax: a decoder whose sublayers stand between two norms, x <- x + norm1b(mixer(norm1(x)));
x <- x + norm2b(ffn(norm2(x))), the norms being of the kind that takes no statistics (tanh(alpha x) w + b).  A layer's
mixer is one of
  `attention`         differential attention (two softmax maps a head over the same values, map 1 - lambda map 2, over
                      its root mean square, times 1 - diff) with interleaved rotary pairs on the first channels of every
                      map of q and k, each query seeing the keys of its own block of `mask.size` positions;
  `latent_attention`  causal attention whose queries come through a normed latent and whose keys and values come from
                      one normed latent a token plus one rotated key part the heads share, every head's output times
                      one sigmoid gate;
  `delta`             the gated delta rule with ONE decay a head behind short causal convolutions, its read-out normed
                      per head and gated by silu of a full projection;
its feed-forward a mixture of gated silu experts chosen by sigmoid scores plus a stored correction, weighted by the
plain scores over their sum times `router.scale`, or none.  `loop` {start, stop, times} runs the layers start .. stop-1
`times` times in a row on the same tensors, every pass against caches and states of its own, and adds the embedding's
output to the stream again before every pass but the first.  The output is the final norm, the embedding table as the
head, and a tanh cap on the logits.  This class knows the config.json keys and the tensor names and nothing else:
every size and constant goes through a spec to a registered part.

config.json: `architecture` (the name), `vocab`, `width`, `norm.eps`, `logit_softcap`, optionally `loop`, and `layers`,
a list of {`type`, `mixer`: sizes and constants, `mlp`: null or {`kind`: moe, `expert.ff`, `router.experts`,
`router.top`, `router.scale`}}.  Positions are not bounded by the model; `max_positions`, when a file gives it, bounds
what the engine plans for.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

from .pamunex import _mask, _object
from .registry import ConfigError, register_architecture
from .specs import (DeltaRuleSpec, DiffAttentionSpec, HeadSpec, LatentAttentionSpec, LayerRun, LayerSpec, ModelSpec, NormSpec,
                    PositionSpec, RoutedMlpSpec)
from .taletar import DEFAULT_MAX_POSITIONS, _freeze, _int, _num, _thaw

DELTA_UNIT_EPS = 1e-6          # inside the root that makes q and k of the delta rule unit vectors


def _rotation(m, where, limit, dims=None):
    """Interleaved pairs over the first `rot.dims` channels (of a map, or of the rotated part, whose size `dims` then
    is what `rot.dims` must say, or may leave to it)."""
    rot = _object(m, "rot", where)
    n = dims if dims is not None and rot.get("dims") is None else _int(rot, "dims", where + "rot.")
    if n % 2 != 0 or n > limit or (dims is not None and n != dims):
        raise ConfigError(f"config.json: {where}rot.dims {n} must be even, at most {limit}" +
                          (f" and equal rot_dim {dims}" if dims is not None else ""))
    return PositionSpec("rope", n, _num(rot, "base", where + "rot.", positive=True), interleaved=True)


def _heads(m, where):
    heads, kv = _int(m, "heads", where), _int(m, "kv_heads", where)
    if heads % kv != 0:
        raise ConfigError(f"config.json: {where}heads {heads} is no multiple of kv_heads {kv}")
    return heads, kv


def _attention(m, width, eps, where):
    heads, kv = _heads(m, where)
    dim = _int(m, "dim", where)
    diff = _num(m, "diff", where)
    return DiffAttentionSpec(kind="diff_attention", hidden=width, q_heads=heads, kv_heads=kv, head_dim=dim,
                             value_dim=_int(m, "vdim", where), scale=_num(m, "scale", where), lam_init=diff,
                             out_scale=1.0 - diff, eps=eps, softcap=None, q_temperature=None, gate=None,
                             position=_rotation(m, where, dim), mask=_mask(m, "chunk", where))


def _latent_attention(m, width, eps, where):
    rot_dim = _int(m, "rot_dim", where)
    return LatentAttentionSpec(kind="latent_attention", hidden=width, heads=_int(m, "heads", where),
                               head_dim=_int(m, "dim", where), rot_dim=rot_dim, value_dim=_int(m, "vdim", where),
                               rank=_int(m, "kv_rank", where), scale=_num(m, "scale", where), eps=eps,
                               position=_rotation(m, where, rot_dim, dims=rot_dim), mask=None, sink=False,
                               q_rank=_int(m, "q_rank", where), head_gate="sigmoid")


def _delta(m, width, eps, where):
    heads, kv = _heads(m, where)
    return DeltaRuleSpec(kind="delta_rule", hidden=width, heads=heads, kv_heads=kv, head_dim=_int(m, "dim", where),
                         value_dim=_int(m, "vdim", where), conv_taps=_int(m, "conv", where), eps=eps,
                         unit_eps=DELTA_UNIT_EPS, decay="head", gate="silu")


def _mlp(mlp, width, where):
    if mlp is None:
        return None
    if not isinstance(mlp, dict) or mlp.get("kind") != "moe":
        raise ConfigError(f"config.json: {where} must be null or an object of kind `moe`")
    router = _object(mlp, "router", where + ".")
    experts, top = _int(router, "experts", where + ".router."), _int(router, "top", where + ".router.")
    if top > experts:
        raise ConfigError(f"config.json: {where}.router: {top} choices among {experts} experts")
    return RoutedMlpSpec("routed_mlp", width, _int(_object(mlp, "expert", where + "."), "ff", where + ".expert."), experts,
                         top, 1, 1, "silu", "sigmoid", True, gated=True, correction=True,
                         route_scale=_num(router, "scale", where + ".router.", default=1.0))


_MIXERS = {"attention": _attention, "latent_attention": _latent_attention, "delta": _delta}
_NORM_PARTS = {"norm1": "norm1", "norm1_after": "norm1b", "norm2": "norm2", "norm2_after": "norm2b"}
_NORM_TENSORS = {"weight": "", "bias": ".b", "alpha": ".alpha"}


@register_architecture("Budorax")
@dataclass(frozen=True)
class BudoraxConfig:
    vocab: int
    width: int
    eps: float
    layers: Tuple                        # the `layers` list of config.json, frozen
    logit_softcap: Optional[float] = None
    loop: Tuple[int, int, int] = (0, 0, 1)      # (start, stop, times)
    max_positions: int = DEFAULT_MAX_POSITIONS
    eos_token_ids: Tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, data):
        for key in ("vocab", "width", "norm", "layers"):
            if key not in data:
                raise ConfigError(f"config.json: missing `{key}`")
        if not isinstance(data["norm"], dict):
            raise ConfigError("config.json: `norm` must be an object with `eps`")
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
        loop = (0, 0, 1)
        if data.get("loop") is not None:
            lp = _object(data, "loop", "")
            loop = (_int(lp, "start", "loop.", lo=0, hi=len(layers)), _int(lp, "stop", "loop.", lo=0, hi=len(layers)),
                    _int(lp, "times", "loop.", lo=1))
            if loop[0] > loop[1]:
                raise ConfigError(f"config.json: loop.start {loop[0]} lies behind loop.stop {loop[1]}")
        cap = data.get("logit_softcap")
        eos = data.get("eos_token_id")
        eos_ids = () if eos is None else (eos,) if isinstance(eos, int) else tuple(eos)
        return cls(vocab=_int(data, "vocab", ""), width=width, eps=_num(data["norm"], "eps", "norm.", positive=True),
                   layers=_freeze(layers), logit_softcap=None if cap is None else _num(data, "logit_softcap", "", positive=True),
                   loop=loop,
                   max_positions=_int(data, "max_positions", "") if "max_positions" in data else DEFAULT_MAX_POSITIONS,
                   eos_token_ids=eos_ids)

    def to_dict(self):
        out = {"architecture": self.architecture, "layers": _thaw(self.layers), "norm": {"eps": self.eps},
               "vocab": self.vocab, "width": self.width}
        if self.logit_softcap is not None:
            out["logit_softcap"] = self.logit_softcap
        if self.loop != (0, 0, 1):
            out["loop"] = {"start": self.loop[0], "stop": self.loop[1], "times": self.loop[2]}
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            out["max_positions"] = self.max_positions
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out

    # ---- the model as parts -------------------------------------------------------------------
    def run_order(self):
        """[(layer, whether the embedding's output joins the stream before it)] in the order the layers run."""
        start, stop, times = self.loop
        n = len(self.layers)
        order = [(i, False) for i in range(start)]
        for p in range(times if stop > start else 0):
            order += [(i, p > 0 and i == start) for i in range(start, stop)]
        return order + [(i, False) for i in range(stop, n)]

    def model_spec(self):
        norm = NormSpec("tanh_norm", self.width, self.eps)
        specs = []
        for i, layer in enumerate(_thaw(self.layers)):
            mixer = _MIXERS[layer["type"]](layer["mixer"], self.width, self.eps, f"layers[{i}].mixer.")
            ffn = _mlp(layer.get("mlp"), self.width, f"layers[{i}].mlp")
            second = None if ffn is None else norm
            specs.append(LayerSpec("sandwich", norm, mixer, second, ffn, norm1_after=norm, norm2_after=second))
        # every run has a cache entry of its own: a looped layer keeps what each of its passes saw
        schedule = tuple(LayerRun(layer, run, add_embedding=again) for run, (layer, again) in enumerate(self.run_order()))
        return ModelSpec(architecture=self.architecture, vocab_size=self.vocab, hidden=self.width, layers=tuple(specs),
                         schedule=schedule, final_norm=norm, tie_embeddings=True, max_positions=self.max_positions,
                         eos_token_ids=self.eos_token_ids,
                         head=HeadSpec("capped_head", self.vocab, self.width, tied=True, softcap=self.logit_softcap))

    # ---- tensor names ----------------------------------------------------------------------------
    @staticmethod
    def global_tensor_name(local):
        return {"embed.weight": "embed", "final_norm.weight": "final.norm", "final_norm.bias": "final.norm.b",
                "final_norm.alpha": "final.norm.alpha", "head.weight": "head"}[local]

    @staticmethod
    def layer_tensor_name(layer, part, local):
        if part in _NORM_PARTS:
            return f"l{layer}.{_NORM_PARTS[part]}{_NORM_TENSORS[local]}"
        return f"l{layer}.{'mix' if part == 'mixer' else 'mlp'}.{local}"
