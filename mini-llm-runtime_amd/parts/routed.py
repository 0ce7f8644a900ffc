"""A mixture of experts with group-limited routing.  Every token scores all experts, s = sigmoid(router . x) in
32-bit (an ordinary product with float output); the experts form equal groups of neighbours, a group's score is the sum of its two largest s, and only
experts of the best groups can be chosen; of those the `top` largest s win and weigh their experts' outputs (as
they are, or divided by their sum, and times `route_scale`).  With `correction` the choice goes by s plus a stored
number an expert while the weights stay the plain s.  An expert is an ungated feed-forward down(act(up(x))) or,
`gated`, down(act(gate(x)) * up(x)).

The step's (token, expert) pairs are sorted by expert on the device, so that every expert's rows lie side by side
and ONE launch multiplies all of them with their own weights (`Kernels.experts_gemm`, the rows of the first product
gathered through the sorted list); nothing of it is read on the host, so a step can be captured."""
from __future__ import annotations

import torch

from ..weights.loader import WeightSpec, stacked
from .mlp import ACTIVATIONS
from .registry import PartError, register_part


@register_part("ffn", "routed_mlp")
class RoutedMlp:
    graph_safe = True

    def __init__(self, spec):
        s = self.spec = spec
        self.gated = bool(getattr(s, "gated", False))
        if self.gated:
            if s.activation not in ("silu", "gelu_tanh"):
                raise PartError(f"gated experts: activation {s.activation!r} is not built (silu, gelu_tanh)")
        elif s.activation not in ACTIVATIONS:
            raise PartError(f"activation {s.activation!r} is not built ({', '.join(ACTIVATIONS)})")
        if s.score != "sigmoid":
            raise PartError("routing: sigmoid scores are what is built")
        self.correction = None
        self.fused_gate = False
        if s.experts % s.group_count != 0 or not 1 <= s.group_keep <= s.group_count or \
                not 1 <= s.top <= s.group_keep * (s.experts // s.group_count):
            raise PartError(f"routing: {s.experts} experts in {s.group_count} groups of which {s.group_keep} stay cannot "
                            f"give {s.top} choices")
        self.router = self.up = self.down = None

    def weight_specs(self):
        s = self.spec
        # (a matrix like the others: its products with the layer's input are exact in 32 bits, and so are their sums'
        # partial results up to rounding: the logits are an ordinary product with float output)
        specs = {"router": WeightSpec((s.experts, s.hidden), init=("normal", 0.0, 0.05))}
        if getattr(s, "correction", False):
            specs["correction"] = WeightSpec((s.experts,), keep_float32=True, init=("normal", 0.0, 0.05))
        for e in range(s.experts):
            if self.gated:                      # (an expert's gate and up side by side: one product gives both)
                specs[f"e{e}.gate"] = WeightSpec((s.intermediate, s.hidden), stack="up")
            specs[f"e{e}.up"] = WeightSpec((s.intermediate, s.hidden), stack="up")
        for e in range(s.experts):
            specs[f"e{e}.down"] = WeightSpec((s.hidden, s.intermediate), stack="down")
        return specs

    def bind(self, weights):
        s = self.spec
        self.router = weights["router"]
        self.correction = weights.get("correction")
        first = [weights[f"e{e}.{n}"] for e in range(s.experts) for n in (("gate", "up") if self.gated else ("up",))]
        self.up = stacked(first).view(s.experts, (2 if self.gated else 1) * s.intermediate, s.hidden)
        # where the grouped product can apply the gate itself, an expert's gate and up rows are laid out in turn, 16
        # and 16: in place when the stack is the loader's memory (an expert at a time: no second copy of the weights;
        # the tensors are marked, so that a second model over the same tensors does not turn them again)
        self.fused_gate = self.gated and self.up.dtype == torch.bfloat16 and s.intermediate % 16 == 0
        if self.fused_gate:
            first_tensor = weights["e0.gate"]
            in_place = self.up.data_ptr() == first_tensor.data_ptr()
            if not (in_place and getattr(first_tensor, "_rows_in_turn", False)):
                for e in range(s.experts):
                    both = self.up[e].clone().view(2, s.intermediate // 16, 16, s.hidden)
                    self.up[e].view(s.intermediate // 16, 2, 16, s.hidden).copy_(both.transpose(0, 1))
                if in_place:
                    first_tensor._rows_in_turn = True
        self.down = stacked([weights[f"e{e}.down"] for e in range(s.experts)]).view(s.experts, s.hidden, s.intermediate)

    def libraries(self):
        return ["gemm", "grouped_gemm"] + (["elementwise"] if self.gated else [])

    def workspace_plan(self, rows, dtype, limits):
        s = self.spec
        pairs = rows * s.top
        return {("route_logits", torch.float32): rows * s.experts, ("route_ids", torch.int32): pairs,
                ("route_weights", torch.float32): pairs,
                ("route_offsets", torch.int32): s.experts + 1, ("route_token", torch.int32): pairs,
                ("route_row", torch.int32): pairs, ("route_act", dtype): pairs * s.intermediate,
                **({("route_gate_up", dtype): pairs * 2 * s.intermediate} if self.gated else {}),
                ("route_y", dtype): pairs * s.hidden, ("ffn_out", dtype): rows * s.hidden}

    def forward(self, ctx, x):
        s = self.spec
        m = x.shape[0]
        k, ws = ctx.kernels, ctx.workspace
        pairs = m * s.top
        ids = ws.get("route_ids", (m, s.top), torch.int32)
        weights = ws.get("route_weights", (m, s.top), torch.float32)
        offsets = ws.get("route_offsets", (s.experts + 1,), torch.int32)
        token_of = ws.get("route_token", (pairs,), torch.int32)
        row_of = ws.get("route_row", (pairs,), torch.int32)
        logits = ws.get("route_logits", (m, s.experts), torch.float32)
        k.gemm(x, self.router, logits)                   # 32-bit sums of the engine's element type's products
        k.router_topk(logits, ids, weights, s.group_count, s.group_keep, correction=self.correction,
                      renormalize=bool(s.renormalize), scale=float(getattr(s, "route_scale", 1.0)))
        k.route_sort(ids, s.experts, offsets, token_of, row_of)
        act = ws.get("route_act", (pairs, s.intermediate), x.dtype)
        if self.fused_gate:
            k.experts_gemm(x, self.up, act, offsets, gather=token_of, act="gated_" + s.activation)
        elif self.gated:
            both = ws.get("route_gate_up", (pairs, 2 * s.intermediate), x.dtype)
            k.experts_gemm(x, self.up, both, offsets, gather=token_of)
            k.gated_act_mul(both, act, s.activation)
        else:
            k.experts_gemm(x, self.up, act, offsets, gather=token_of, act=s.activation)
        y = ws.get("route_y", (pairs, s.hidden), x.dtype)
        k.experts_gemm(act, self.down, y, offsets)
        out = ws.get("ffn_out", (m, s.hidden), x.dtype)
        k.route_combine(y, row_of, weights, out)
        return out
