"""Taletar: a decoder whose layers each pick one of three mixers -- differential attention, gated linear
attention, Mamba-2 -- beside an optional clamped gated feed-forward, both reading the same input:
x <- x + (mixer(norm1(x)) + ffn(norm2(x))).  This class knows the config.json keys and the tensor names
and nothing else: every size and constant goes through a spec to a registered part.

config.json: `architecture` (the name), `vocab`, `width`, `norm.eps`, and `layers`, a list of
{`type`: attention | gla | mamba2, `mixer`: the mixer's sizes and constants, `mlp`: null or
{`kind`: dense, `ff`, `limit`}}.  Positions are not bounded by the model (no rotation, no table);
`max_positions`, when a file gives it, bounds what the engine plans for, else `DEFAULT_MAX_POSITIONS` does.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Tuple

from .registry import ConfigError, register_architecture
from .specs import (ClampedGluSpec, DiffAttentionSpec, GlaSpec, LayerRun, LayerSpec, Mamba2Spec, ModelSpec, NormSpec,
                    QueryTemperature)

DEFAULT_MAX_POSITIONS = 1 << 20
_LIMIT = 1_000_000


def _int(d, key, where, lo=1, hi=_LIMIT):
    v = d.get(key)
    if isinstance(v, bool) or not isinstance(v, int) or not lo <= v <= hi:
        raise ConfigError(f"config.json: {where}`{key}` must be an integer in {lo}..{hi}, got {v!r}")
    return v


def _num(d, key, where, positive=False, default=None):
    v = d.get(key, default)
    if isinstance(v, bool) or not isinstance(v, (int, float)) or not math.isfinite(v) or (positive and v <= 0):
        raise ConfigError(f"config.json: {where}`{key}` must be a finite{' positive' if positive else ''} number, got {v!r}")
    return float(v)


def _freeze(value):
    """A JSON value as something hashable, so that the configuration stays a frozen dataclass."""
    if isinstance(value, dict):
        return tuple((k, _freeze(v)) for k, v in value.items())
    if isinstance(value, list):
        return tuple(_freeze(v) for v in value)
    return value


def _thaw(value):
    if isinstance(value, tuple) and all(isinstance(v, tuple) and len(v) == 2 and isinstance(v[0], str) for v in value) \
            and value:
        return {k: _thaw(v) for k, v in value}
    if isinstance(value, tuple):
        return [_thaw(v) for v in value]
    return value


@register_architecture("Taletar")
@dataclass(frozen=True)
class TaletarConfig:
    vocab: int
    width: int
    eps: float
    layers: Tuple            # the `layers` list of config.json, frozen
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
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") != "dense":
                    raise ConfigError(f"config.json: {where}mlp must be null or an object of kind `dense`")
                _int(mlp, "ff", where + "mlp.")
                _num(mlp, "limit", where + "mlp.", positive=True)
        eos = data.get("eos_token_id")
        eos_ids = () if eos is None else (eos,) if isinstance(eos, int) else tuple(eos)
        return cls(vocab=_int(data, "vocab", ""), width=width, eps=_num(data["norm"], "eps", "norm.", positive=True),
                   layers=_freeze(layers),
                   max_positions=_int(data, "max_positions", "") if "max_positions" in data else DEFAULT_MAX_POSITIONS,
                   eos_token_ids=eos_ids)

    def to_dict(self):
        out = {"architecture": self.architecture, "layers": _thaw(self.layers), "norm": {"eps": self.eps},
               "vocab": self.vocab, "width": self.width}
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            out["max_positions"] = self.max_positions
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out

    # ---- the model as parts -------------------------------------------------------------------
    def model_spec(self):
        norm = NormSpec("rmsnorm", self.width, self.eps)
        specs = []
        for i, layer in enumerate(_thaw(self.layers)):
            mixer = _MIXERS[layer["type"]](layer["mixer"], self.width, self.eps, f"layers[{i}].mixer.")
            mlp = layer.get("mlp")
            ffn = None if mlp is None else ClampedGluSpec("clamped_glu", self.width, mlp["ff"], float(mlp["limit"]))
            specs.append(LayerSpec("parallel", norm, mixer, None if ffn is None else norm, ffn))
        n = len(specs)
        return ModelSpec(architecture=self.architecture, vocab_size=self.vocab, hidden=self.width, layers=tuple(specs),
                         schedule=tuple(LayerRun(i, i) for i in range(n)), final_norm=norm, tie_embeddings=False,
                         max_positions=self.max_positions, eos_token_ids=self.eos_token_ids)

    # ---- tensor names ----------------------------------------------------------------------------
    @staticmethod
    def global_tensor_name(local):
        return {"embed.weight": "embed", "final_norm.weight": "final.norm", "head.weight": "head"}[local]

    @staticmethod
    def layer_tensor_name(layer, part, local):
        if part in ("norm1", "norm2"):
            return f"l{layer}.{part}"
        return f"l{layer}.{'mix' if part == 'mixer' else 'mlp'}.{local}"


def _attention(m, width, eps, where):
    heads, kv = _int(m, "heads", where), _int(m, "kv_heads", where)
    if heads % kv != 0:
        raise ConfigError(f"config.json: {where}heads {heads} is no multiple of kv_heads {kv}")
    temp = m.get("q_temp")
    if temp is not None:
        if not isinstance(temp, dict):
            raise ConfigError(f"config.json: {where}q_temp must be an object with `coef` and `every`")
        temp = QueryTemperature(_num(temp, "coef", where + "q_temp."), _num(temp, "every", where + "q_temp.", positive=True))
    diff = _num(m, "diff", where)
    cap = m.get("softcap")
    return DiffAttentionSpec(
        kind="diff_attention", hidden=width, q_heads=heads, kv_heads=kv, head_dim=_int(m, "dim", where),
        value_dim=_int(m, "vdim", where), scale=_num(m, "scale", where), lam_init=diff, out_scale=1.0 - diff, eps=eps,
        softcap=None if cap is None else _num(m, "softcap", where, positive=True), q_temperature=temp, gate="sigmoid")


def _gla(m, width, eps, where):
    return GlaSpec(kind="gla", hidden=width, heads=_int(m, "heads", where), head_dim=_int(m, "dim", where),
                   value_dim=_int(m, "vdim", where), decay_rank=m.get("rank") or 0, tau=_num(m, "tau", where, positive=True),
                   eps=eps)


def _mamba2(m, width, eps, where):
    heads, groups = _int(m, "heads", where), _int(m, "groups", where)
    if heads % groups != 0:
        raise ConfigError(f"config.json: {where}heads {heads} is no multiple of groups {groups}")
    parts = _int(m, "norm_groups", where)
    inner = heads * _int(m, "vdim", where)
    if inner % parts != 0:
        raise ConfigError(f"config.json: {where}norm_groups {parts} does not divide heads * vdim = {inner}")
    return Mamba2Spec(kind="mamba2", hidden=width, heads=heads, value_dim=m["vdim"], state=_int(m, "state", where),
                      groups=groups, conv_taps=_int(m, "conv", where), norm_groups=parts, eps=eps)


_MIXERS = {"attention": _attention, "gla": _gla, "mamba2": _mamba2}
