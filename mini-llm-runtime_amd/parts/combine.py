"""Several mixers side by side on the same input: out = sum_i scale_i * mixer_i(x).  The mixers are registered parts
like any other, built from their own specs; each keeps a cache entry of its own (pages for one, a state of fixed size
for another), its tensors are named `<name>.<its local name>`, and the weighted sum of their outputs is taken in
32-bit."""
from __future__ import annotations

from dataclasses import replace

from .registry import PartError, build_part, register_part


@register_part("mixer", "mixer_sum")
class MixerSum:
    def __init__(self, spec):
        self.spec = spec
        if len(spec.mixers) < 2:
            raise PartError("a sum of mixers needs at least two")
        self.names = [name for name, _, _ in spec.mixers]
        if len(set(self.names)) != len(self.names) or any("." in n or not n for n in self.names):
            raise PartError(f"the mixers of a sum need distinct plain names, got {self.names}")
        self.scales = [float(scale) for _, _, scale in spec.mixers]
        self.mixers = [build_part("mixer", sub) for _, sub, _ in spec.mixers]
        for i, mixer in enumerate(self.mixers):
            if not hasattr(mixer, "out_name"):
                raise PartError(f"mixer {self.names[i]!r} cannot write to a buffer of its own (`out_name`)")
            mixer.out_name = f"mixer_out_{i}"
        self.graph_safe = all(getattr(m, "graph_safe", False) for m in self.mixers)

    def weight_specs(self):
        specs = {}
        for name, mixer in zip(self.names, self.mixers):
            for local, ws in mixer.weight_specs().items():
                specs[f"{name}.{local}"] = replace(ws, stack=f"{name}.{ws.stack}") if ws.stack is not None else ws
        return specs

    def bind(self, weights):
        for name, mixer in zip(self.names, self.mixers):
            prefix = name + "."
            mixer.bind({local[len(prefix):]: t for local, t in weights.items() if local.startswith(prefix)})

    def cache_spec(self):
        """One entry per mixer, in their order: the model hands `forward` as many cache ids."""
        return tuple(mixer.cache_spec() for mixer in self.mixers)

    def libraries(self):
        names = {"elementwise"}
        for mixer in self.mixers:
            names.update(mixer.libraries())
        return sorted(names)

    def check_limits(self, *args):
        for mixer in self.mixers:
            if hasattr(mixer, "check_limits"):
                mixer.check_limits(*args)

    def workspace_plan(self, rows, dtype, limits):
        plan = {("mixer_out", dtype): rows * self.spec.hidden}
        for mixer in self.mixers:
            if hasattr(mixer, "workspace_plan"):
                for key, count in mixer.workspace_plan(rows, dtype, limits).items():
                    plan[key] = max(plan.get(key, 0), count)
        return plan

    def forward(self, ctx, x, cache_id, write_cache=True):
        if not isinstance(cache_id, tuple) or len(cache_id) != len(self.mixers):
            raise PartError("a sum of mixers needs one cache id for each of them")
        outs = [mixer.forward(ctx, x, cid, write_cache) for mixer, cid in zip(self.mixers, cache_id)]
        out = ctx.workspace.get("mixer_out", tuple(outs[0].shape), x.dtype)
        k = ctx.kernels
        k.scaled_sum(outs[0], outs[1], out, self.scales[0], self.scales[1])
        for extra, scale in zip(outs[2:], self.scales[2:]):
            k.scaled_sum(out, extra, out, 1.0, scale)
        return out
