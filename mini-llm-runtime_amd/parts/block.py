"""Arrangement of the parts in a layer.  Pre-norm residual block (src/minillm/runtime.cpp:245-337):
h += mixer(norm1(h)); h += ffn(norm2(h)).  The residual stream h is float; every add into it is
fused with the norm that follows, so a block hands its last output on as `pending` instead of
adding it itself.  `norm2` and `ffn` may be missing: a layer of the first sublayer only.
Other arrangements: mixer and feed-forward side by side (`parallel`), norms behind the sublayers (`postnorm`), norms in
front of AND behind each sublayer (`sandwich`)."""
from __future__ import annotations

from .registry import Complete, Handoff, build_part, register_part


@register_part("block", "prenorm")
class PreNormBlock:
    graph_safe = True        # forward launches kernels over the step's device vectors only
    def __init__(self, spec):
        self.norm1 = build_part("norm", spec.norm1)
        self.mixer = build_part("mixer", spec.mixer)
        if (spec.ffn is None) != (spec.norm2 is None):
            raise ValueError("a pre-norm block has a feed-forward and its norm, or neither")
        self.norm2 = build_part("norm", spec.norm2) if spec.norm2 is not None else None
        self.ffn = build_part("ffn", spec.ffn) if spec.ffn is not None else None

    def parts(self):
        out = {"norm1": self.norm1, "mixer": self.mixer}
        if self.ffn is not None:
            out.update(norm2=self.norm2, ffn=self.ffn)
        return out

    def workspace_plan(self, rows, dtype, limits):
        import torch
        width = self.norm1.size
        few = min(rows, 16)
        return {("normed", dtype): rows * width, ("handoff_x", dtype): few * width,
                ("handoff_ss", torch.float32): few * max(1, (width + 15) // 16)}

    def forward(self, ctx, h, pending, cache_id, write_cache=True, next_norm=None):
        fusable = lambda norm: norm is not None and getattr(norm, "fusable_rmsnorm", False) and norm.size == h.shape[1]
        if (ctx.kernels.handoff_supported(h.shape[0]) and fusable(self.norm1) and fusable(self.norm2)
                and getattr(self.mixer, "forward_handoff", None) is not None
                and getattr(self.ffn, "forward_handoff", None) is not None):
            # few rows: every norm is shared between the projection before it (which adds into h and leaves
            # h * weight and partial sums of squares) and the projection after it (which applies the scale)
            hand = pending if isinstance(pending, Handoff) and pending.norm is self.norm1 else \
                self.norm1.prenorm(ctx, h, None if isinstance(pending, Complete) else pending)
            hand = self.mixer.forward_handoff(ctx, hand, h, self.norm2, cache_id, write_cache)
            return self.ffn.forward_handoff(ctx, hand, h, next_norm if fusable(next_norm) else None)
        if isinstance(pending, Complete):                 # h is complete already
            pending = None
        normed = ctx.workspace.get("normed", tuple(h.shape), ctx.dtype)
        self.norm1.forward(ctx, h, pending, normed)
        mixed = self.mixer.forward(ctx, normed, cache_id, write_cache)
        if self.ffn is None:
            return mixed                                  # (whoever norms next adds it)
        self.norm2.forward(ctx, h, mixed, normed)
        return self.ffn.forward(ctx, normed)


@register_part("block", "parallel")
class ParallelBlock:
    """Mixer and feed-forward side by side on the same input, each behind a norm of its own:
    h += mixer(norm1(h)) + ffn(norm2(h)); the sum of the two branches is taken in 32-bit and added to the float
    residual stream.  `norm2` and `ffn` may be missing (a layer without a feed-forward).  Both norms divide by
    the same root mean square, so one pass over h serves both (`Kernels.add2_rmsnorm2`), and that pass is the
    one that adds the branches of the block before: a block ends by norming h for the block that follows
    (`Normed`) when that one is of this kind too, else it adds its branches itself."""
    graph_safe = True
    wants_next_block = True

    def __init__(self, spec):
        self.norm1 = build_part("norm", spec.norm1)
        self.mixer = build_part("mixer", spec.mixer)
        if (spec.ffn is None) != (spec.norm2 is None):
            raise ValueError("a parallel block has a feed-forward and its norm, or neither")
        self.norm2 = build_part("norm", spec.norm2) if spec.norm2 is not None else None
        self.ffn = build_part("ffn", spec.ffn) if spec.ffn is not None else None

    def parts(self):
        out = {"norm1": self.norm1, "mixer": self.mixer}
        if self.ffn is not None:
            out.update(norm2=self.norm2, ffn=self.ffn)
        return out

    def workspace_plan(self, rows, dtype, limits):
        width = self.norm1.size
        return {("normed", dtype): rows * width, ("normed2", dtype): rows * width}

    def _one_pass(self, width):
        """Whether the block's norms are plain RMSNorms over the whole width with one eps: then they share a pass."""
        norms = [self.norm1] + ([self.norm2] if self.norm2 is not None else [])
        return all(getattr(n, "fusable_rmsnorm", False) and n.size == width and n.eps == self.norm1.eps for n in norms)

    def _norm_into(self, ctx, h, d1, d2, x1, x2):
        """h += d1 + d2 (either may be None); x1 = norm1(h), x2 = norm2(h)."""
        k = ctx.kernels
        if self._one_pass(h.shape[1]):
            k.add2_rmsnorm2(h, d1, d2, self.norm1.weight, self.norm2.weight if self.norm2 is not None else None,
                            x1, x2 if self.norm2 is not None else None, self.norm1.eps)
            return
        if d2 is not None:
            k.residual_add2(h, d1, d2)
            d1 = None
        self.norm1.forward(ctx, h, d1, x1)
        if self.norm2 is not None:
            self.norm2.forward(ctx, h, None, x2)

    def forward(self, ctx, h, pending, cache_id, write_cache=True, next_norm=None, next_block=None):
        from .registry import Normed
        shape = tuple(h.shape)
        x1 = ctx.workspace.get("normed", shape, ctx.dtype)
        x2 = ctx.workspace.get("normed2", shape, ctx.dtype) if self.ffn is not None else None
        if isinstance(pending, Normed) and pending.norms == ((self.norm1, self.norm2) if self.ffn is not None else (self.norm1,)):
            x1, x2 = pending.outputs if self.ffn is not None else (pending.outputs[0], None)
        else:
            self._norm_into(ctx, h, None if isinstance(pending, Complete) else pending, None, x1, x2)
        mixed = self.mixer.forward(ctx, x1, cache_id, write_cache)
        fed = self.ffn.forward(ctx, x2) if self.ffn is not None else None
        if isinstance(next_block, ParallelBlock) and next_block._one_pass(h.shape[1]):
            # the branches are added and h is normed for the next block in one pass (its inputs go where this
            # block's own were: both branches have read them)
            n1 = ctx.workspace.get("normed", shape, ctx.dtype)
            n2 = ctx.workspace.get("normed2", shape, ctx.dtype) if next_block.ffn is not None else None
            next_block._norm_into(ctx, h, mixed, fed, n1, n2)
            return Normed((next_block.norm1, next_block.norm2) if next_block.ffn is not None else (next_block.norm1,),
                          (n1, n2) if next_block.ffn is not None else (n1,))
        if fed is None:
            return mixed                                  # (one delta: whoever norms next adds it)
        ctx.kernels.residual_add2(h, mixed, fed)
        return None


@register_part("block", "postnorm")
class PostNormBlock:
    """The norms stand behind the sublayers: h += norm1(mixer(h)); h += norm2(ffn(h)).  Mixer and feed-forward read
    the residual stream itself (in the engine's element type), and what they give is normed and added to the float
    stream in one pass, which also leaves the stream for the next reader (`LayerNorm.add_into`).  `norm2` and `ffn`
    may be missing (a layer without a feed-forward)."""
    graph_safe = True

    def __init__(self, spec):
        self.norm1 = build_part("norm", spec.norm1)
        self.mixer = build_part("mixer", spec.mixer)
        if (spec.ffn is None) != (spec.norm2 is None):
            raise ValueError("a post-norm block has a feed-forward and its norm, or neither")
        self.norm2 = build_part("norm", spec.norm2) if spec.norm2 is not None else None
        self.ffn = build_part("ffn", spec.ffn) if spec.ffn is not None else None
        for norm in (self.norm1, self.norm2):
            if norm is not None and not hasattr(norm, "add_into"):
                raise ValueError("a post-norm block needs norms that can add into the stream (`add_into`)")

    def parts(self):
        out = {"norm1": self.norm1, "mixer": self.mixer}
        if self.ffn is not None:
            out.update(norm2=self.norm2, ffn=self.ffn)
        return out

    def workspace_plan(self, rows, dtype, limits):
        import torch
        return {("stream", dtype): rows * self.norm1.size} if dtype != torch.float32 else {}

    def forward(self, ctx, h, pending, cache_id, write_cache=True, next_norm=None):
        import torch
        from .registry import Streamed
        k = ctx.kernels
        narrow = ctx.dtype != torch.float32          # (the float engine's sublayers read h itself)
        x = h
        if narrow:
            x = ctx.workspace.get("stream", tuple(h.shape), ctx.dtype)
        if isinstance(pending, Streamed) and (not narrow or pending.x is x):
            pass                                          # the block before left the stream where we read it
        else:
            if pending is not None and not isinstance(pending, Complete):
                k.residual_add(h, pending)
            if narrow:
                k.cast_rows(h, x)
        mixed = self.mixer.forward(ctx, x, cache_id, write_cache)
        last = self.ffn is None
        self.norm1.add_into(ctx, mixed, h, cast=x if narrow and not (last and next_norm is None) else None)
        if not last:
            fed = self.ffn.forward(ctx, x)
            self.norm2.add_into(ctx, fed, h, cast=x if narrow and next_norm is not None else None)
        return Streamed(x) if next_norm is not None else None


@register_part("block", "sandwich")
class SandwichBlock:
    """A norm in front of and one behind each sublayer: h += norm1_after(mixer(norm1(h))); h += norm2_after(ffn(norm2(h))).
    The norm behind a sublayer, the residual sum and the norm in front of the next sublayer are one pass over the
    stream where the norms can (`add_into(..., then=, out=)`: the norm without statistics); `norm2`, `ffn` and
    `norm2_after` may be missing.  `extra` (a float matrix like h) is added to the stream with the block's last
    sublayer, before the next block's norm."""
    graph_safe = True
    adds_extra = True

    def __init__(self, spec):
        self.norm1 = build_part("norm", spec.norm1)
        self.mixer = build_part("mixer", spec.mixer)
        if spec.norm1_after is None:
            raise ValueError("a sandwich block needs the norm behind its mixer")
        self.norm1_after = build_part("norm", spec.norm1_after)
        if not ((spec.ffn is None) == (spec.norm2 is None) == (spec.norm2_after is None)):
            raise ValueError("a sandwich block has a feed-forward and both its norms, or none of the three")
        self.norm2 = build_part("norm", spec.norm2) if spec.norm2 is not None else None
        self.ffn = build_part("ffn", spec.ffn) if spec.ffn is not None else None
        self.norm2_after = build_part("norm", spec.norm2_after) if spec.norm2_after is not None else None
        for norm in (self.norm1_after, self.norm2_after):
            if norm is not None and not hasattr(norm, "add_into"):
                raise ValueError("a sandwich block needs norms behind its sublayers that can add into the stream (`add_into`)")

    def parts(self):
        out = {"norm1": self.norm1, "mixer": self.mixer, "norm1_after": self.norm1_after}
        if self.ffn is not None:
            out.update(norm2=self.norm2, ffn=self.ffn, norm2_after=self.norm2_after)
        return out

    def workspace_plan(self, rows, dtype, limits):
        return {("normed", dtype): rows * self.norm1.size}

    @staticmethod
    def _same_pass(after, then):
        """Whether `after.add_into` can take the norm `then` in its pass: both of one kind that offers it."""
        return then is not None and type(then) is type(after) and hasattr(then, "params")

    def forward(self, ctx, h, pending, cache_id, write_cache=True, next_norm=None, extra=None):
        from .registry import Normed
        normed = ctx.workspace.get("normed", tuple(h.shape), ctx.dtype)
        if isinstance(pending, Normed) and pending.norms == (self.norm1,):
            x = pending.outputs[0]                       # the block before normed the stream for this one
        else:
            self.norm1.forward(ctx, h, None if isinstance(pending, Complete) else pending, normed)
            x = normed
        mixed = self.mixer.forward(ctx, x, cache_id, write_cache)
        if self.ffn is None:
            return self._last(ctx, h, mixed, self.norm1_after, next_norm, extra, normed)
        if self._same_pass(self.norm1_after, self.norm2):
            self.norm1_after.add_into(ctx, mixed, h, then=self.norm2, out=normed)
        else:
            self.norm1_after.add_into(ctx, mixed, h)
            self.norm2.forward(ctx, h, None, normed)
        fed = self.ffn.forward(ctx, normed)
        return self._last(ctx, h, fed, self.norm2_after, next_norm, extra, normed)

    def _last(self, ctx, h, delta, after, next_norm, extra, normed):
        """The block's last sublayer into the stream; the next block's first norm in the same pass where it can be."""
        from .registry import Normed
        if self._same_pass(after, next_norm) and next_norm.size == h.shape[1]:
            after.add_into(ctx, delta, h, extra=extra, then=next_norm, out=normed)
            return Normed((next_norm,), (normed,))
        if extra is not None:
            after.add_into(ctx, delta, h, extra=extra)
        else:
            after.add_into(ctx, delta, h)
        return None
