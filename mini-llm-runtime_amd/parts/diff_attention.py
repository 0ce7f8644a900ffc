"""Differential attention over the paged cache.  Every query head holds two maps: two softmax attentions with
queries and keys of their own over the same values; the head's output is map 1 - lam * map 2 with
lam = exp(lq1 . lk1) - exp(lq2 . lk2) + lam_init (one number a layer), divided by its root mean square over the
value channels, times `out_scale`, times sigmoid of the head's gate; then the output projection.  Query and key
channels of a map (`head_dim`) and value channels (`value_dim`) are sizes of their own; consecutive query heads
share a kv head.  A query's position may enter as a factor on it (`QueryTemperature`) and a score may be squashed by
`softcap * tanh(score / softcap)`; with a position part, the first channels of every map of q and k are turned by
the token's position before the keys are cached; position p sees keys 0..p, or what a mask rule leaves of them
(the last `size` positions, or the positions of p's own block of `size`).

Per token the cache keeps the keys of both maps [kv_heads, 2 * head_dim] and the values [kv_heads, value_dim]
(`PagedSpec`).  q, k, v and the gate are one stacked projection of the mixer's input.

The float engine runs every token through the scalar kernel with key ranges of one width (the same bits however a
request is cut or batched); the bfloat16 engine takes prompt portions and single tokens to the matrix-core kernel
where it takes the sizes, a token's keys cut into ranges where the batch alone would not fill the GPU."""
from __future__ import annotations

import math

import torch

from ..cache.manager import PAGE, PagedSpec
from ..weights.loader import WeightSpec, stacked
from .registry import PartError, build_part, register_part
from .sink_attention import _mask_of, _rope_table

PARTIAL_CAP = 32 << 20        # floats that the key ranges' partial results of one launch may take at most
SMALL_GROUP = 4               # tokens: a request that brings more of them to a step is a prompt portion


@register_part("mixer", "diff_attention")
class DiffAttention:
    graph_safe = True        # forward launches kernels over the step's device vectors only

    def __init__(self, spec):
        s = self.spec = spec
        if s.q_heads % s.kv_heads != 0:
            raise PartError(f"q_heads {s.q_heads} is no multiple of kv_heads {s.kv_heads}")
        if not 1 <= s.head_dim <= 256 or not 1 <= s.value_dim <= 256:
            raise PartError(f"head_dim {s.head_dim} / value_dim {s.value_dim}: the attention kernels take sizes up to 256")
        if s.gate not in (None, "sigmoid"):
            raise PartError(f"gate {s.gate!r} is not built (sigmoid or none)")
        self.mask, self.mask_size = _mask_of(s) if getattr(s, "mask", None) is not None else (None, 0)
        self.position = build_part("position", s.position) if getattr(s, "position", None) is not None else None
        self.q_width, self.k_width = s.q_heads * 2 * s.head_dim, s.kv_heads * 2 * s.head_dim
        self.v_width, self.o_width = s.kv_heads * s.value_dim, s.q_heads * s.value_dim
        self.proj = self.o = None
        self.lam = None
        self._partial_floats = PARTIAL_CAP
        self._page_size = 16

    def weight_specs(self):
        s = self.spec
        small = ("normal", 0.0, 0.1)
        specs = {"q": WeightSpec((self.q_width, s.hidden), stack="qkvg"), "k": WeightSpec((self.k_width, s.hidden), stack="qkvg"),
                 "v": WeightSpec((self.v_width, s.hidden), stack="qkvg")}
        if s.gate is not None:
            specs["g"] = WeightSpec((self.o_width, s.hidden), stack="qkvg")
        specs["o"] = WeightSpec((s.hidden, self.o_width))
        for name in ("lq1", "lk1", "lq2", "lk2"):
            specs[name] = WeightSpec((s.head_dim,), keep_float32=True, init=small)
        return specs

    def bind(self, weights):
        s = self.spec
        self.proj = stacked([weights[n] for n in ("q", "k", "v") + (("g",) if s.gate is not None else ())])
        self.o = weights["o"]
        # lam is one number a layer: computed once, in 32-bit, when the weights are bound
        f = lambda n: weights[n].detach().to("cpu", torch.float32).numpy()
        one = f("lq1") * f("lk1")
        two = f("lq2") * f("lk2")
        import numpy as np
        self.lam = float(np.exp(one.sum(dtype=np.float32)) - np.exp(two.sum(dtype=np.float32)) + np.float32(s.lam_init))

    def cache_spec(self):
        s = self.spec
        # (values transposed within a page: the keys of one channel side by side, as the matrix cores want them)
        return PagedSpec((("k", (s.kv_heads, PAGE, 2 * s.head_dim)), ("v", (s.kv_heads, s.value_dim, PAGE))),
                         self.mask_size if self.mask is not None else None)

    def libraries(self):
        return ["gemm", "diff_attention"]

    @staticmethod
    def _splits(max_context, split_keys):
        """(width of a key range, number of ranges): ranges of `split_keys` keys at absolute positions, whatever
        the batch; beyond 1024 ranges the width doubles (the merge's limit)."""
        if split_keys <= 0 or max_context <= split_keys:
            return 0, 1
        keys = split_keys
        while -(-max_context // keys) > 1024:
            keys *= 2
        return keys, -(-max_context // keys)

    def workspace_plan(self, rows, dtype, limits):
        from ..kernels.ops import Kernels
        s = self.spec
        _, splits = self._splits(limits["max_length"], limits["split_keys"])
        per_row = Kernels.diff_partial_numel(1, s.q_heads, s.value_dim, splits)
        total = self.q_width + self.k_width + self.v_width + (self.o_width if s.gate is not None else 0)
        self._partial_floats = max(per_row, min(rows * per_row, PARTIAL_CAP))
        plan = {("diff_proj", dtype): rows * total, ("attn", dtype): rows * self.o_width,
                ("mixer_out", dtype): rows * s.hidden,
                ("diff_partial", torch.float32): max(per_row, min(rows * per_row, PARTIAL_CAP))}
        for factor in (4, 8, 16):
            plan[(f"token_groups_{SMALL_GROUP}_{factor}", torch.int32)] = 2 * rows + 2
        return plan

    def _tile_splits(self, ctx, units, places, budget):
        """(width of a key range, number of ranges) for a launch of the matrix-core kernel that has `units`
        workgroups without ranges and `places` rows of partial results: no ranges where the batch fills the GPU or
        the context is short; else the widest ranges that still give `target_workgroups`, widened further until
        the partial results fit `budget` floats."""
        s = self.spec
        base, longest = ctx.split_keys, ctx.max_context
        # keys that one workgroup walks without ranges: every earlier key, or behind a mask its tokens' window or block
        # (ranges stay absolute, [s * keys, (s + 1) * keys): those that lie before a token's first key stay empty)
        walk = longest if self.mask is None else min(longest, self.mask_size + 64 + 128)
        reach = ctx.kernels.diff_tiles_reach(self._page_size)       # the most keys one workgroup walks
        forced = walk > reach
        if base <= 0 and forced:
            raise PartError(f"a context of {longest} tokens needs key ranges (split_keys > 0): one workgroup walks {reach} keys")
        if base <= 0 or walk <= base or (units >= ctx.target_workgroups and not forced):
            return 0, 1
        keys = base
        while keys * 2 < walk and keys * 2 <= reach and (units * (-(-walk // (keys * 2))) >= ctx.target_workgroups or
                                                          (forced and units >= ctx.target_workgroups)):
            keys *= 2
        numel = lambda k: ctx.kernels.diff_partial_numel(places, s.q_heads, s.value_dim, -(-longest // k))
        while (numel(keys) > budget or -(-longest // keys) > 1024) and keys < longest and keys * 2 <= reach:
            keys *= 2
        splits = -(-longest // keys)
        return (keys, splits) if splits > 1 else (0, 1)

    def _attend_tiles(self, ctx, q, gate, view, attn):
        """The bfloat16 engine on the matrix cores: prompt portions in groups of 16 to 64 tokens, single tokens and
        portions of up to SMALL_GROUP tokens in groups of their own."""
        s = self.spec
        k = ctx.kernels
        tokens = k.diff_tiles_group_tokens(s.q_heads, s.kv_heads)
        self._page_size = view.page_size
        small, big, _ = ctx.token_groups(SMALL_GROUP, tokens // SMALL_GROUP)
        temp = s.q_temperature
        g = s.q_heads // s.kv_heads
        per_group = s.kv_heads * (-(-g // min(4, g)))
        partial = ctx.workspace.get("diff_partial", (self._partial_floats,), torch.float32)
        for (first, count, n), group_tokens in ((big, tokens), (small, SMALL_GROUP)):
            if n == 0:
                continue
            split_keys, splits = self._tile_splits(ctx, n * per_group, n * group_tokens, partial.numel())
            # (single tokens and short portions always leave partial results, where their room allows: the two maps
            # of a head then run side by side and the merge kernel finishes the head)
            through = splits > 1 or (group_tokens == SMALL_GROUP and
                                     k.diff_partial_numel(n * group_tokens, s.q_heads, s.value_dim, 1) <= partial.numel())
            k.diff_attention_tiles(q, view.tensors["k"], view.tensors["v"], view.block_table, ctx.slots, ctx.positions, gate,
                                   attn, partial if through else None, first, count, n, group_tokens, s.q_heads, s.kv_heads, s.head_dim,
                                   s.value_dim, view.page_size, float(s.scale), self.lam, float(s.out_scale), float(s.eps),
                                   softcap=s.softcap, temp_coef=temp.coef if temp else 0.0,
                                   temp_every=temp.every if temp else 1.0, split_keys=split_keys, max_splits=splits,
                                   max_context=ctx.max_context, mask=self.mask, mask_size=self.mask_size)

    def forward(self, ctx, x, cache_id, write_cache=True):
        s = self.spec
        k = ctx.kernels
        m = x.shape[0]
        proj = ctx.workspace.get("diff_proj", (m, self.proj.shape[0]), x.dtype)
        k.gemm(x, self.proj, proj)
        a = self.q_width
        b = a + self.k_width
        c = b + self.v_width
        q, keys, values = proj[:, :a], proj[:, a:b], proj[:, b:c]
        gate = proj[:, c:] if s.gate is not None else None
        view = ctx.cache.paged_view(cache_id)
        k_pages, v_pages = view.tensors["k"], view.tensors["v"]
        if self.position is not None:
            rope, interleaved = _rope_table(self.position, ctx, x.device, s.head_dim)
            k.diff_qkv_prep(q, keys, values, k_pages, v_pages, view.block_table, ctx.slots, ctx.positions, rope, s.q_heads,
                            s.kv_heads, s.head_dim, s.value_dim, view.page_size, write_cache, interleaved=interleaved)
        elif write_cache:
            k.diff_kv_write(keys, values, k_pages, v_pages, view.block_table, ctx.slots, ctx.positions, s.kv_heads,
                            s.head_dim, s.value_dim, view.page_size)
        attn = ctx.workspace.get("attn", (m, self.o_width), x.dtype)
        if k.diff_tiles_supported(s.q_heads, s.kv_heads, s.head_dim, s.value_dim, view.page_size, proj.stride(0), proj.stride(0)) \
                and a % 8 == 0 and c % 4 == 0:
            self._attend_tiles(ctx, q, gate, view, attn)
            out = ctx.workspace.get("mixer_out", (m, s.hidden), x.dtype)
            k.gemm(attn, self.o, out)
            return out
        split_keys, splits = self._splits(ctx.max_context, ctx.split_keys)
        per_row = k.diff_partial_numel(1, s.q_heads, s.value_dim, splits)
        chunk = max(1, min(m, PARTIAL_CAP // per_row))
        partial = ctx.workspace.get("diff_partial", (chunk * per_row,), torch.float32)
        temp = s.q_temperature
        for r0 in range(0, m, chunk):
            r1 = min(m, r0 + chunk)
            k.diff_attention(q[r0:r1], k_pages, v_pages, view.block_table, ctx.slots[r0:r1], ctx.positions[r0:r1],
                             gate[r0:r1] if gate is not None else None, attn[r0:r1], partial, s.q_heads, s.kv_heads,
                             s.head_dim, s.value_dim, view.page_size, float(s.scale), self.lam, float(s.out_scale),
                             float(s.eps), softcap=s.softcap, temp_coef=temp.coef if temp else 0.0,
                             temp_every=temp.every if temp else 1.0, split_keys=split_keys, max_splits=splits,
                             mask=self.mask, mask_size=self.mask_size)
        out = ctx.workspace.get("mixer_out", (m, s.hidden), x.dtype)
        k.gemm(attn, self.o, out)
        return out
