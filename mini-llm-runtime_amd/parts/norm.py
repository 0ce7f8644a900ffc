"""RMSNorm: y = (x * rsqrt(mean(x^2) + eps)) * w, the weight multiplying directly
(src/minillm/kernels.cpp:209-216).  The residual add that precedes a norm in the layer is
fused into the same kernel.  A spec with a `weight_offset` stores its weight as the factor's distance from
that offset (a weight "around zero": factor 1 + w); the factor is formed once, in 32-bit, when the weights are bound."""
from __future__ import annotations

import torch

from ..weights.loader import WeightSpec
from .registry import register_part


@register_part("norm", "rmsnorm")
class RmsNorm:
    graph_safe = True        # forward launches kernels over the step's device vectors only
    fusable_rmsnorm = True   # the projections before and after it may share this norm between them (weight, eps as here)
    def __init__(self, spec):
        self.size, self.eps = spec.size, float(spec.eps)
        self.offset = float(getattr(spec, "weight_offset", 0.0))
        self.weight = None

    def weight_specs(self):
        init = ("normal", 0.0, 0.1) if self.offset != 0.0 else None
        return {"weight": WeightSpec((self.size,), keep_float32=True, init=init)}

    def bind(self, weights):
        self.weight = weights["weight"] if self.offset == 0.0 else (weights["weight"].float() + self.offset).contiguous()

    def libraries(self):
        return ["elementwise"]

    def prenorm(self, ctx, h, delta):
        """h += delta (delta may be None) and the first half of this norm for the projection that follows:
        a `Handoff` (see parts/registry.py)."""
        from .registry import Handoff
        m = h.shape[0]
        x = ctx.workspace.get("handoff_x", (m, self.size), ctx.dtype)
        ss = ctx.workspace.get("handoff_ss", (m, 1), torch.float32)
        ctx.kernels.rows_prenorm(h, delta, self.weight, x, ss)
        return Handoff(self, x, ss)

    def forward(self, ctx, h, delta, out, rows=None, write_h=True):
        ctx.kernels.add_rmsnorm(h, delta, self.weight, out, self.eps, rows=rows, write_h=write_h)
        return out


@register_part("norm", "tanh_norm")
class TanhNorm:
    """A norm that takes no mean and no variance: y = tanh(alpha x) * weight + bias, element by element, with one
    learned number alpha a norm; 32-bit.  It serves in front of a sublayer (`forward`, on the residual stream) and
    behind one (`add_into`: the norm of what the sublayer gave is added to the stream, and the norm in front of the
    next sublayer may be taken in the same pass)."""
    graph_safe = True

    def __init__(self, spec):
        self.size = spec.size
        self.weight = self.bias = None
        self.alpha = 1.0

    def weight_specs(self):
        return {"weight": WeightSpec((self.size,), keep_float32=True),
                "bias": WeightSpec((self.size,), keep_float32=True, init=("normal", 0.0, 0.1)),
                "alpha": WeightSpec((), keep_float32=True, init=("uniform", 0.3, 1.0))}

    def bind(self, weights):
        self.weight, self.bias = weights["weight"], weights["bias"]
        self.alpha = float(weights["alpha"].detach().to("cpu", torch.float32).reshape(()))    # (one number, read once)

    def libraries(self):
        return ["elementwise"]

    def params(self):
        return self.weight, self.bias, self.alpha

    def forward(self, ctx, h, delta, out, rows=None, write_h=True):
        ctx.kernels.tanh_norm_rows(h, delta, self.weight, self.bias, self.alpha, out, rows=rows, write_h=write_h)
        return out

    def add_into(self, ctx, delta, h, extra=None, then=None, out=None):
        """h += norm(delta) (+ extra, a float matrix like h); `then` (another norm of this kind) with `out`: out =
        then(h) in the same pass."""
        ctx.kernels.tanh_norm_add(delta, self.weight, self.bias, self.alpha, h, extra=extra,
                                  then=then.params() if then is not None else None, out=out)


@register_part("norm", "layernorm")
class LayerNorm:
    """y = (x - mean) / sqrt(var + eps) * weight + bias, var the mean of the squared deviations; 32-bit."""
    graph_safe = True

    def __init__(self, spec):
        self.size, self.eps = spec.size, float(spec.eps)
        self.weight = self.bias = None

    def weight_specs(self):
        return {"weight": WeightSpec((self.size,), keep_float32=True),
                "bias": WeightSpec((self.size,), keep_float32=True, init=("normal", 0.0, 0.1))}

    def bind(self, weights):
        self.weight, self.bias = weights["weight"], weights["bias"]

    def libraries(self):
        return ["elementwise"]

    def forward(self, ctx, h, delta, out, rows=None, write_h=True, out_scale=1.0):
        """The norm of the residual stream itself (a model's final norm): x = h + delta (delta may be None; it is
        added into h), out[r] = norm(x[rows[r] or r])."""
        if delta is not None:
            ctx.kernels.residual_add(h, delta)
        ctx.kernels.layernorm_rows(h, self.weight, self.bias, out, self.eps, rows=rows, out_scale=out_scale)
        return out

    def add_into(self, ctx, delta, h, cast=None):
        """h += norm(delta): the norm of what a sublayer gave, added to the float residual stream in the same pass;
        `cast` (the engine's element type) receives the new h as the next sublayer's input."""
        ctx.kernels.layernorm_add(delta, self.weight, self.bias, h, cast=cast, eps=self.eps)
