"""SwiGLU feed-forward: out = (silu(x Wgate^T) * (x Wup^T)) Wdown^T with silu(g) = g / (1 + exp(-g))
(src/minillm/runtime.cpp:323-336).  Gate and up are one stacked projection.  The gate's activation is the spec's:
silu, or gelu_tanh (0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3)))); for few rows either rides on the projection,
the norm handed between projections is silu's alone."""
from __future__ import annotations

import torch

from ..weights.loader import WeightSpec, stacked
from .registry import Handoff, PartError, register_part


@register_part("ffn", "swiglu")
class SwiGluMlp:
    graph_safe = True        # forward launches kernels over the step's device vectors only
    def __init__(self, spec):
        if spec.activation not in ("silu", "gelu_tanh"):
            raise PartError(f"activation {spec.activation!r} is not built (silu, gelu_tanh)")
        self.spec = spec
        self.gate_up = None
        self.down = None
        if spec.activation != "silu":         # the projections' fused epilogues are silu's
            self.forward_handoff = None

    def weight_specs(self):
        s = self.spec
        return {"gate_proj": WeightSpec((s.intermediate, s.hidden), stack="gate_up"),
                "up_proj": WeightSpec((s.intermediate, s.hidden), stack="gate_up"),
                "down_proj": WeightSpec((s.hidden, s.intermediate))}

    def bind(self, weights):
        self.gate_up = stacked([weights["gate_proj"], weights["up_proj"]])
        self.down = weights["down_proj"]

    def libraries(self):
        return ["gemm", "elementwise"]

    def workspace_plan(self, rows, dtype, limits):
        s = self.spec
        return {("act", dtype): rows * s.intermediate, ("gate_up", dtype): rows * 2 * s.intermediate,
                ("ffn_out", dtype): rows * s.hidden}

    def forward_handoff(self, ctx, hand, h, norm_after):
        """As `forward` on the norm that `hand` describes, its scale applied inside the first projection; the
        second projection adds into h and prepares `norm_after` (None: nothing follows)."""
        s = self.spec
        m = h.shape[0]
        k = ctx.kernels
        act = ctx.workspace.get("act", (m, s.intermediate), ctx.dtype)
        k.gemm_prenormed(hand.x, hand.ss, hand.norm.eps, self.gate_up, act, gated=True)
        if norm_after is None:
            k.gemm_residual(act, self.down, h)
            return None
        x = ctx.workspace.get("handoff_x", (m, s.hidden), ctx.dtype)
        ss = ctx.workspace.get("handoff_ss", (m, k.handoff_parts(s.hidden)), torch.float32)
        k.gemm_residual(act, self.down, h, norm_after.weight, x, ss)
        return Handoff(norm_after, x, ss)

    def forward(self, ctx, x):
        s = self.spec
        m = x.shape[0]
        act = ctx.workspace.get("act", (m, s.intermediate), x.dtype)
        if s.activation == "silu" and ctx.kernels.gated_silu_fused(m, s.hidden):
            ctx.kernels.gemm_gated_silu(x, self.gate_up, act)      # few rows: the activation rides on the projection
        elif s.activation == "gelu_tanh" and m <= 64 and ctx.kernels.streams_weight(m, s.hidden):
            ctx.kernels.gemm_gated_gelu_tanh(x, self.gate_up, act)
        else:
            gate_up = ctx.workspace.get("gate_up", (m, 2 * s.intermediate), x.dtype)
            ctx.kernels.gemm(x, self.gate_up, gate_up)
            if s.activation == "silu":
                ctx.kernels.silu_mul(gate_up, act)
            else:
                ctx.kernels.gated_act_mul(gate_up, act, s.activation)
        out = ctx.workspace.get("ffn_out", (m, s.hidden), x.dtype)
        ctx.kernels.gemm(act, self.down, out)
        return out


@register_part("ffn", "clamped_glu")
class ClampedGluMlp:
    """A gated feed-forward whose branches are clamped: g = min(x Wgate^T, limit), u = clamp(x Wup^T, -limit, limit),
    out = (g * sigmoid(slope * g) * (u + 1)) Wdown^T.  Gate and up are one stacked projection."""
    graph_safe = True

    def __init__(self, spec):
        if not spec.limit > 0:
            raise PartError("the clamp's limit must be positive")
        self.spec = spec
        self.gate_up = None
        self.down = None

    def weight_specs(self):
        s = self.spec
        return {"gate": WeightSpec((s.intermediate, s.hidden), stack="gate_up"),
                "up": WeightSpec((s.intermediate, s.hidden), stack="gate_up"),
                "down": WeightSpec((s.hidden, s.intermediate))}

    def bind(self, weights):
        self.gate_up = stacked([weights["gate"], weights["up"]])
        self.down = weights["down"]

    def libraries(self):
        return ["gemm", "elementwise"]

    def workspace_plan(self, rows, dtype, limits):
        s = self.spec
        return {("act", dtype): rows * s.intermediate, ("gate_up", dtype): rows * 2 * s.intermediate,
                ("ffn_out", dtype): rows * s.hidden}

    def forward(self, ctx, x):
        s = self.spec
        m = x.shape[0]
        k = ctx.kernels
        act = ctx.workspace.get("act", (m, s.intermediate), x.dtype)
        if k.streams_weight(m, s.hidden):             # few rows: the activation rides on the projection
            k.gemm_gated_clamped(x, self.gate_up, act, float(s.limit), float(s.slope))
        else:
            gate_up = ctx.workspace.get("gate_up", (m, 2 * s.intermediate), x.dtype)
            k.gemm(x, self.gate_up, gate_up)
            k.clamped_glu(gate_up, act, float(s.limit), float(s.slope))
        out = ctx.workspace.get("ffn_out", (m, s.hidden), x.dtype)
        k.gemm(act, self.down, out)
        return out


ACTIVATIONS = ("relu_squared",)


@register_part("ffn", "plain_mlp")
class PlainMlp:
    """down(act(up(x))) without a gate; act = relu(x)^2."""
    graph_safe = True

    def __init__(self, spec):
        if spec.activation not in ACTIVATIONS:
            raise PartError(f"activation {spec.activation!r} is not built ({', '.join(ACTIVATIONS)})")
        self.spec = spec
        self.up = self.down = None

    def weight_specs(self):
        s = self.spec
        return {"up": WeightSpec((s.intermediate, s.hidden)), "down": WeightSpec((s.hidden, s.intermediate))}

    def bind(self, weights):
        self.up, self.down = weights["up"], weights["down"]

    def libraries(self):
        return ["gemm", "elementwise"]

    def workspace_plan(self, rows, dtype, limits):
        s = self.spec
        return {("act", dtype): rows * s.intermediate, ("ffn_out", dtype): rows * s.hidden}

    def forward(self, ctx, x):
        s = self.spec
        m = x.shape[0]
        k = ctx.kernels
        act = ctx.workspace.get("act", (m, s.intermediate), x.dtype)
        k.gemm(x, self.up, act)
        k.relu_squared(act, act)
        out = ctx.workspace.get("ffn_out", (m, s.hidden), x.dtype)
        k.gemm(act, self.down, out)
        return out
