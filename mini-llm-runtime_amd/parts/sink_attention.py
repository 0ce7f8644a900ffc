"""Two mixers whose softmax has a sink -- one more summand exp(sink[head]) in the denominator, a learned number a
head that stands for no key and brings no value -- and whose queries see the keys that a mask rule names: the last
`size` positions (`window`) or the positions of the query's own block of `size` (`chunk`), counted from the
request's first token.

`SinkAttention`: grouped-query attention with query/key and value sizes of their own, optional biases on q, k, v,
a norm per head of q and k before the rotation (or after it; with a weight shared by the heads or without one), a
rotation of a head's first channels (how many, their pairing and the angles are the position part's), and
optionally a gate on the heads' outputs (sigmoid(Wg x), before the output projection).  Per token the cache keeps
keys [kv_heads, head_dim] and values [kv_heads, value_dim], both row-major.  The sink may be left out: the usual
softmax.

`LatentAttention`: keys and values of all heads are up-projections of ONE normed latent vector a token, plus one
rotated key part that all heads share; only the latent vector and that part are cached, [rank + rot_dim] a token.
The up-projections are moved to the query's side: q_lat[h] = W_uk[h]^T q_plain[h], so a head's score is
q_lat[h] . latent + q_rot[h] . k_rot -- attention of all heads over ONE shared key row whose first `rank` channels
are also the value -- and the head's output is W_uv[h] applied to the attention's latent result.  With `q_rank` the
queries come through a normed latent of their own, q = W_uq norm(W_dq x).  With `head_gate` every head's output is
multiplied by ONE number, sigmoid(Wg x)[head], before the output projection.
"""
from __future__ import annotations

import torch

from ..cache.manager import PAGE, PagedSpec
from ..weights.loader import WeightSpec, stacked
from .registry import PartError, build_part, register_part


def _mask_of(spec):
    if spec.mask is None:
        return None, 0
    if spec.mask.kind not in ("window", "chunk") or spec.mask.size < 1:
        raise PartError(f"mask {spec.mask.kind!r} of size {spec.mask.size}: window or chunk, of a positive size")
    return spec.mask.kind, int(spec.mask.size)


def _rope_table(position, ctx, device, rot_limit):
    """(the position part's table, whether its pairs are interleaved), or (None, False) without a rotation."""
    if position is None:
        return None, False
    rotation = position.rotation(ctx.max_positions, device)
    if rotation is None:
        return None, False
    if rotation.dim % 2 != 0 or not 2 <= rotation.dim <= rot_limit or rotation.table.shape[1] != rotation.dim:
        raise PartError(f"the position part turns {rotation.dim} channels: must be even, at most {rot_limit}")
    return rotation.table, bool(rotation.interleaved)


PARTIAL_CAP = 8 << 20         # floats that the shares of the key ranges of one launch may take at most
RANGE_KEYS = 128              # the narrowest key range of a workgroup
MOST_RANGES = 16              # key ranges of a group at most


def _groups_plan(rows, q_heads, kv_heads, value_dim):
    """The token-group vectors and the room for key ranges' shares that `attend` asks the step's context for."""
    from ..kernels.ops import Kernels
    _, big_tokens, _, small_tokens = Kernels.sink_tiles_layout(q_heads, kv_heads)
    return {(f"token_groups_{small_tokens}_{max(1, big_tokens // small_tokens)}", torch.int32): 2 * rows + 2,
            ("sink_partial", torch.float32): min(PARTIAL_CAP, Kernels.sink_partial_numel(rows, small_tokens, q_heads, value_dim, MOST_RANGES))}


def _key_ranges(ctx, groups, tokens, workgroups, q_heads, value_dim, mask, mask_size):
    """(keys a range, ranges, room for their shares) for a launch over `groups` groups of single tokens or short portions
    that has `workgroups` workgroups without ranges: where those do not fill the GPU, a group's keys (its window or
    chunk; without a mask the step's longest context) are dealt out to several workgroups, as many as reach
    `target_workgroups`, none narrower than RANGE_KEYS, and no more than their shares have room for."""
    k = ctx.kernels
    reach = (mask_size if mask == "chunk" else mask_size + tokens - 1) if mask is not None else ctx.max_context
    reach = min(reach, ctx.max_context + 31) + 31             # (ranges start at the first tile, which may start earlier)
    most = max(1, min(MOST_RANGES, -(-reach // RANGE_KEYS), -(-ctx.target_workgroups // max(1, workgroups))))
    room = ctx.workspace.get("sink_partial", (min(PARTIAL_CAP, k.sink_partial_numel(groups, tokens, q_heads, value_dim, most)),),
                             torch.float32)
    most = min(most, room.numel() // k.sink_partial_numel(groups, tokens, q_heads, value_dim, 1))
    if most <= 1:
        return 0, 1, None
    keys = -(-(-(-reach // most)) // 32) * 32
    return keys, -(-reach // keys), room


def attend(ctx, q, k_pages, v_pages, view, sink, out, q_heads, kv_heads, key_dim, value_dim, scale, mask, mask_size):
    """Every token of the step over the keys it sees.  The bfloat16 engine on the matrix cores where they take the
    sizes (prompt portions in workgroups of 64 columns, single tokens and short portions in workgroups of 16 whose
    wavefronts share the value channels); else, and in the float engine, one wavefront a (token, head), whose sums
    follow from the token's position alone."""
    k = ctx.kernels
    if k.sink_tiles_supported(key_dim, value_dim, k_pages.shape[3], v_pages.shape[3], view.page_size, mask, mask_size,
                              ctx.max_positions) and q.shape[1] % 8 == 0:
        big_heads, big_tokens, small_heads, small_tokens = k.sink_tiles_layout(q_heads, kv_heads)
        small, big, _ = ctx.token_groups(small_tokens, max(1, big_tokens // small_tokens))
        for (first, count, n), heads, split in ((big, big_heads, False), (small, small_heads, True)):
            if n == 0:
                continue
            keys, ranges, room = (0, 1, None)
            if split:
                per_group = kv_heads * -(-(q_heads // kv_heads) // heads)
                keys, ranges, room = _key_ranges(ctx, n, small_tokens, n * per_group, q_heads, value_dim, mask, mask_size)
            k.sink_attention_tiles(q, k_pages, v_pages, view.block_table, ctx.slots, ctx.positions, sink, out, first,
                                   count, n, heads, split, q_heads, kv_heads, key_dim, value_dim, view.page_size,
                                   scale, mask, mask_size, ctx.max_positions, partial=room, split_keys=keys, splits=ranges)
        return
    k.sink_attention(q, k_pages, v_pages, view.block_table, ctx.slots, ctx.positions, sink, out, q_heads, kv_heads,
                     key_dim, value_dim, view.page_size, scale, mask, mask_size)


@register_part("mixer", "sink_attention")
class SinkAttention:
    graph_safe = True

    def __init__(self, spec):
        s = self.spec = spec
        if s.q_heads % s.kv_heads != 0:
            raise PartError(f"q_heads {s.q_heads} is no multiple of kv_heads {s.kv_heads}")
        self.mask, self.mask_size = _mask_of(s)
        if s.qk_norm is not None and s.qk_norm.size != s.head_dim:
            raise PartError("the q/k norm must span one head")
        self.position = build_part("position", s.position) if s.position is not None else None
        self.q_width, self.k_width, self.v_width = s.q_heads * s.head_dim, s.kv_heads * s.head_dim, s.kv_heads * s.value_dim
        self.o_width = s.q_heads * s.value_dim
        if s.gate not in (None, "sigmoid", "silu"):
            raise PartError(f"gate {s.gate!r}: sigmoid, silu or none")
        self.norm_order = None if s.qk_norm is None else "after" if s.qk_norm_after_rotation else "before"
        self.out_name = "mixer_out"                      # (a part that runs several mixers gives each a buffer of its own)
        self.qkv = self.o = self.bias = self.q_norm = self.k_norm = self.sink = None

    def weight_specs(self):
        s = self.spec
        specs = {"q": WeightSpec((self.q_width, s.hidden), stack="qkv"), "k": WeightSpec((self.k_width, s.hidden), stack="qkv"),
                 "v": WeightSpec((self.v_width, s.hidden), stack="qkv"), "o": WeightSpec((s.hidden, self.o_width))}
        if s.gate is not None:                           # (behind q, k, v: one projection gives all four)
            specs["g"] = WeightSpec((self.o_width, s.hidden), stack="qkv")
        if s.bias:
            for name, width in (("q.b", self.q_width), ("k.b", self.k_width), ("v.b", self.v_width)):
                specs[name] = WeightSpec((width,), keep_float32=True, init=("normal", 0.0, 0.02))
        if s.qk_norm is not None and s.qk_norm_weight:
            specs["q.norm"] = WeightSpec((s.head_dim,), keep_float32=True)
            specs["k.norm"] = WeightSpec((s.head_dim,), keep_float32=True)
        if s.sink:
            specs["sink"] = WeightSpec((s.q_heads,), keep_float32=True, init=("normal", 0.0, 1.0))
        return specs

    def bind(self, weights):
        s = self.spec
        self.qkv = stacked([weights[n] for n in (("q", "k", "v", "g") if s.gate is not None else ("q", "k", "v"))])
        self.o = weights["o"]
        self.bias = torch.cat([weights["q.b"], weights["k.b"], weights["v.b"]]).contiguous() if s.bias else None
        if s.qk_norm is not None and s.qk_norm_weight:
            self.q_norm, self.k_norm = weights["q.norm"], weights["k.norm"]
        self.sink = weights["sink"] if s.sink else None

    def cache_spec(self):
        s = self.spec
        return PagedSpec((("k", (s.kv_heads, PAGE, s.head_dim)), ("v", (s.kv_heads, PAGE, s.value_dim))),
                         self.mask_size if self.mask is not None else None)

    def libraries(self):
        return ["gemm", "sink_attention", "elementwise"]

    def workspace_plan(self, rows, dtype, limits):
        s = self.spec
        gate = self.o_width if s.gate is not None else 0
        return {("sink_proj", dtype): rows * (self.q_width + self.k_width + self.v_width + gate), ("q", dtype): rows * self.q_width,
                ("attn", dtype): rows * self.o_width, (self.out_name, dtype): rows * s.hidden,
                **_groups_plan(rows, s.q_heads, s.kv_heads, s.value_dim)}

    def forward(self, ctx, x, cache_id, write_cache=True):
        s = self.spec
        k = ctx.kernels
        m = x.shape[0]
        proj = ctx.workspace.get("sink_proj", (m, self.qkv.shape[0]), x.dtype)
        k.gemm(x, self.qkv, proj)
        view = ctx.cache.paged_view(cache_id)
        k_pages, v_pages = view.tensors["k"], view.tensors["v"]
        q = ctx.workspace.get("q", (m, self.q_width), x.dtype)
        rope, interleaved = _rope_table(self.position, ctx, x.device, s.head_dim)
        qkv_width = self.q_width + self.k_width + self.v_width
        k.sink_qkv_prep(proj, self.bias, q, k_pages, v_pages, view.block_table, ctx.slots, ctx.positions, self.q_norm,
                        self.k_norm, s.qk_norm.eps if s.qk_norm is not None else 0.0, rope, s.q_heads, s.kv_heads,
                        s.head_dim, s.value_dim, view.page_size, write_cache, norm=self.norm_order, interleaved=interleaved)
        attn = ctx.workspace.get("attn", (m, self.o_width), x.dtype)
        attend(ctx, q, k_pages, v_pages, view, self.sink, attn, s.q_heads, s.kv_heads, s.head_dim, s.value_dim,
               float(s.scale), self.mask, self.mask_size)
        if s.gate is not None:
            k.gate_mul(attn, proj[:, qkv_width:], attn, s.gate)
        out = ctx.workspace.get(self.out_name, (m, s.hidden), x.dtype)
        k.gemm(attn, self.o, out)
        return out


@register_part("mixer", "latent_attention")
class LatentAttention:
    graph_safe = True

    def __init__(self, spec):
        s = self.spec = spec
        self.mask, self.mask_size = _mask_of(s)
        if s.position is None or s.position.dim != s.rot_dim or s.rot_dim % 2 != 0:
            raise PartError("latent attention turns its whole rotated part: an even rot_dim with a position part as wide")
        self.position = build_part("position", s.position)
        self.q_width = s.heads * (s.head_dim + s.rot_dim)
        self.row = s.rank + s.rot_dim                    # a token's cache row, and a query head after the move
        self.o_width = s.heads * s.value_dim
        self.out_name = "mixer_out"
        self.head_gate = getattr(s, "head_gate", None)
        if self.head_gate not in (None, "sigmoid"):
            raise PartError(f"head_gate {self.head_gate!r}: sigmoid or none")
        self.proj = self.o = self.norm = self.uk_t = self.uv = self.sink = self.uq = self.q_norm = self.gate = None

    def weight_specs(self):
        s = self.spec
        if s.q_rank is None:
            first = {"q": WeightSpec((self.q_width, s.hidden), stack="down")}
        else:           # the queries' latent comes out of the same projection as the keys' and values'
            first = {"dq": WeightSpec((s.q_rank, s.hidden), stack="down"), "dq.norm": WeightSpec((s.q_rank,), keep_float32=True),
                     "uq": WeightSpec((self.q_width, s.q_rank))}
        specs = {**first, "dkv": WeightSpec((self.row, s.hidden), stack="down"),
                 "dkv.norm": WeightSpec((s.rank,), keep_float32=True),
                 "uk": WeightSpec((s.heads * s.head_dim, s.rank)), "uv": WeightSpec((self.o_width, s.rank)),
                 "o": WeightSpec((s.hidden, self.o_width))}
        if s.sink:
            specs["sink"] = WeightSpec((s.heads,), keep_float32=True, init=("normal", 0.0, 1.0))
        if self.head_gate is not None:      # (with a query latent it rides behind the two latents in the one projection)
            specs["g"] = WeightSpec((s.heads, s.hidden), stack="down" if s.q_rank is not None else None)
        return specs

    def bind(self, weights):
        s = self.spec
        if s.q_rank is None:
            self.proj = stacked([weights["q"], weights["dkv"]])
            self.gate = weights["g"] if self.head_gate is not None else None
        else:
            self.proj = stacked([weights["dq"], weights["dkv"]] + ([weights["g"]] if self.head_gate is not None else []))
            self.uq, self.q_norm = weights["uq"], weights["dq.norm"]
        self.norm = weights["dkv.norm"]
        # the key up-projection as the queries meet it: per head [rank, head_dim]
        self.uk_t = weights["uk"].view(s.heads, s.head_dim, s.rank).transpose(1, 2).contiguous()
        self.uv = weights["uv"].view(s.heads, s.value_dim, s.rank)
        self.o = weights["o"]
        self.sink = weights["sink"] if s.sink else None

    def cache_spec(self):
        return PagedSpec((("latent", (1, PAGE, self.row)),), self.mask_size if self.mask is not None else None)

    def libraries(self):
        return ["gemm", "grouped_gemm", "sink_attention", "elementwise"]

    def workspace_plan(self, rows, dtype, limits):
        s = self.spec
        first = self.q_width if s.q_rank is None else s.q_rank
        more = {} if s.q_rank is None else {("latent_cq", dtype): rows * s.q_rank, ("latent_queries", dtype): rows * self.q_width}
        if self.head_gate is not None:
            more[("latent_gate", dtype)] = rows * s.heads
        return {("latent_proj", dtype): rows * (first + self.row + (s.heads if self.head_gate is not None else 0)),
                ("latent_q", dtype): rows * s.heads * self.row,
                ("latent_out", dtype): rows * s.heads * s.rank, ("attn", dtype): rows * self.o_width,
                (self.out_name, dtype): rows * s.hidden, **more, **_groups_plan(rows, s.heads, 1, s.rank)}

    def forward(self, ctx, x, cache_id, write_cache=True):
        s = self.spec
        k = ctx.kernels
        m = x.shape[0]
        ld = self.proj.shape[0]
        proj = ctx.workspace.get("latent_proj", (m, ld), x.dtype)
        k.gemm(x, self.proj, proj)
        view = ctx.cache.paged_view(cache_id)
        pages = view.tensors["latent"]
        q = ctx.workspace.get("latent_q", (m, s.heads * self.row), x.dtype)
        rope, interleaved = _rope_table(self.position, ctx, x.device, s.rot_dim)
        gate = None
        if s.q_rank is None:
            queries, q_ld = proj, ld
            if self.head_gate is not None:
                gate = ctx.workspace.get("latent_gate", (m, s.heads), x.dtype)
                k.gemm(x, self.gate, gate)
            k.latent_prep(proj, q, pages, view.block_table, ctx.slots, ctx.positions, self.norm, float(s.eps), rope, s.heads,
                          s.head_dim, s.rot_dim, s.rank, view.page_size, write_cache, interleaved=interleaved)
        else:
            # the queries' latent: normed in 32-bit over its own root mean square, then up to the heads
            cq = ctx.workspace.get("latent_cq", (m, s.q_rank), x.dtype)
            k.rmsnorm_columns(proj[:, :s.q_rank], self.q_norm, cq, float(s.eps))
            queries, q_ld = ctx.workspace.get("latent_queries", (m, self.q_width), x.dtype), self.q_width
            k.gemm(cq, self.uq, queries)
            if self.head_gate is not None:
                gate = proj[:, s.q_rank + self.row:]
            k.latent_prep(proj[:, s.q_rank:s.q_rank + self.row], q, pages, view.block_table, ctx.slots, ctx.positions, self.norm, float(s.eps),
                          rope, s.heads, s.head_dim, s.rot_dim, s.rank, view.page_size, write_cache, q_src=queries,
                          interleaved=interleaved)
        # the plain query channels through the key up-projection, head by head, into the first `rank` channels
        k.heads_gemm(torch.as_strided(queries, (m, s.heads, s.head_dim), (q_ld, s.head_dim + s.rot_dim, 1)), self.uk_t,
                     torch.as_strided(q, (m, s.heads, s.rank), (s.heads * self.row, self.row, 1)))
        lat = ctx.workspace.get("latent_out", (m, s.heads * s.rank), x.dtype)
        attend(ctx, q, pages, pages, view, self.sink, lat, s.heads, 1, self.row, s.rank, float(s.scale), self.mask,
               self.mask_size)
        attn = ctx.workspace.get("attn", (m, self.o_width), x.dtype)
        k.heads_gemm(lat.view(m, s.heads, s.rank), self.uv, attn.view(m, s.heads, s.value_dim))
        if gate is not None:
            k.head_gate_mul(attn, gate, attn, s.heads)
        out = ctx.workspace.get(self.out_name, (m, s.hidden), x.dtype)
        k.gemm(attn, self.o, out)
        return out
