"""Attention whose heads exchange their scores before the softmax, over keys that are also the values.

"mixed_attention": H query heads over G key heads (query head h reads key head h // (H/G)) of `dim`
dims.  q and k are rotated by the position part in its first dims and then, with `qk_norm`
"rms_after_rotation", each head is divided by its root mean square (no weight, eps `norm_eps`).
The value of a key is the key as it was projected, before rotation and norm (`values` "keys": there is
no value projection).  raw_g(i, j) = q_g(i) . k(j) * scale; with `head_mix` the scores that enter the
softmax are s_h = sum_g T[h, g] raw_g, T a learned [H, H] tensor.  Position i sees j <= i; with
`chunk` only those j of its own chunk, floor(i / chunk) == floor(j / chunk), counted from position 0 of
the sequence.  `sink`: None, "zero" (the softmax's denominator holds one more term exp(0) that has no
value) or "learned" (one score a head, a tensor).

The cache layer keeps, for a token and key head, the key as it is scored and the key as it was
projected; prompt portions and single tokens read both from there with the same kernel, in tiles of
keys whose place depends on positions only, so that a token's result does not depend on how its
sequence was cut into steps.  In bfloat16, with heads in fours and head sizes in multiples of 32, the
matrix-core kernel runs (rows of a sequence in items of up to 16 that do not cross a chunk's edge);
any other size, and float32, goes through the plain kernel.
"""
from __future__ import annotations

import numpy as np
import torch

from ..config.specs import CacheNeed, MixerSpec
from ..kernels import ops
from ..weights.spec import TensorSpec
from .base import LazyNorm, Mixer, lookup, register_mixer
from .kv_attention import product, tiles_of

_WORKGROUPS_WANTED = 256        # items split their keys until about this many workgroups run (one a CU)
_MOST_SPLITS = 8
_PARTIAL_LIMIT = 64 << 20       # float32 words of the splits' parts
_LAYOUT = "by key head: the keys as scored by slot, then the keys as projected by dimension"


@register_mixer("mixed_attention")
class MixedAttention(Mixer):
    graph_safe = True

    def __init__(self, spec: MixerSpec, prefix: str, dtype: torch.dtype):
        self.prefix, self.dtype = prefix, dtype
        self.hidden = spec.get("hidden")
        self.num_heads = spec.get("num_heads")
        self.kv_heads = spec.get("num_kv_heads", self.num_heads)
        self.dim = spec.get("dim")
        self.scale = float(spec.get("scale", self.dim ** -0.5))
        self.chunk = int(spec.get("chunk", 0) or 0)
        self.sink = spec.get("sink")                       # None | "zero" | "learned"
        self.head_mix = bool(spec.get("head_mix", False))
        self.qk_norm = spec.get("qk_norm")                 # None | "rms_after_rotation"
        self.norm_eps = float(spec.get("norm_eps", 0.0))
        if spec.get("values", "keys") != "keys":
            raise ValueError("mixed_attention takes its values from the keys as projected")
        if self.sink not in (None, "zero", "learned"):
            raise ValueError(f"sink is None, 'zero' or 'learned', not {self.sink!r}")
        if self.qk_norm not in (None, "rms_after_rotation"):
            raise ValueError(f"qk_norm is None or 'rms_after_rotation', not {self.qk_norm!r}")
        if self.num_heads % self.kv_heads:
            raise ValueError(f"{self.num_heads} heads are not a multiple of {self.kv_heads} kv heads")
        if self.chunk < 0:
            raise ValueError("a chunk has a positive size (0: none)")
        self.position = lookup("position", spec.position.kind)(spec.position) if spec.position else None
        if self.position is not None and self.position.pairing != 0:
            raise ValueError("mixed_attention rotates pairs (i, i + half)")
        given = dict(spec.get("names") or ())
        defaults = dict(q="q_proj.weight", k="k_proj.weight", o="o_proj.weight", head_mix="head_mix", sink="sinks")
        self.names = {role: prefix + given.get(role, default) for role, default in defaults.items()}
        self.q_width, self.k_width = self.num_heads * self.dim, self.kv_heads * self.dim
        self.matrix = dtype == torch.bfloat16 and ops.attention_mix_fits(self.num_heads, self.dim) and self.hidden % 8 == 0
        self.items_key = f"mixed_attention.items.{self.chunk}"

    def tensor_specs(self):
        n, H = self.names, self.num_heads
        specs = [TensorSpec(n["q"], (self.q_width, self.hidden)), TensorSpec(n["k"], (self.k_width, self.hidden)),
                 TensorSpec(n["o"], (self.hidden, self.q_width))]
        if self.head_mix:
            specs.append(TensorSpec(n["head_mix"], (H, H), role="vector"))
        if self.sink == "learned":
            specs.append(TensorSpec(n["sink"], (H,), role="vector"))
        return specs

    def bind(self, tensors):
        n = self.names
        self.w_qk = torch.cat([tensors.pop(n["q"]), tensors.pop(n["k"])], dim=0).contiguous()
        self.w_o = tensors.pop(n["o"]).contiguous()
        self.mix = tensors.pop(n["head_mix"]).to(torch.float32).contiguous() if self.head_mix else None
        self.mix_t = self.mix.t().contiguous() if self.mix is not None else None
        self.sinks = tensors.pop(n["sink"]).to(torch.float32).contiguous() if self.sink == "learned" else None
        self.w_qk_tiles, self.w_o_tiles = tiles_of(self.dtype, self.w_qk, self.w_o)

    def cache_spec(self):
        return CacheNeed("full", (self.kv_heads, 2 * self.dim), 0, layout=_LAYOUT)

    def key_layout(self):
        pos = self.position
        return (self.kv_heads, self.dim, self.qk_norm, self.norm_eps, None if pos is None else pos.signature())

    def prepare(self, info):
        if self.position is not None:
            self.position.prepare(info.num_positions, info.device)

    def plan(self, plan):
        """The step's rows in items of up to 16 that stay within a chunk (once a step and chunk size,
        whichever layers ask): first row, rows, first position, block-table row."""
        if not self.matrix or self.items_key in plan.arrays:
            return
        items = []
        for s, seg in enumerate(plan.segments):
            off = 0
            while off < seg.length:
                p = seg.start + off
                room = min(ops.ATTENTION_MIX_ROWS, seg.length - off)
                if self.chunk:
                    room = min(room, self.chunk - p % self.chunk)
                items.append((seg.row0 + off, room, p, s))
                off += room
        plan.add(self.items_key, np.asarray(items, dtype=np.int32).reshape(-1, 4))

    def forward_add(self, ctx, x, h, cache_layer: int, writes_cache: bool):
        hn = h.tensor() if isinstance(h, LazyNorm) else h
        H, G, D = self.num_heads, self.kv_heads, self.dim
        cache = ctx.storage.layer(cache_layer, (G, ctx.page_size * 2 * D))
        tables = ctx.block_tables[ctx.storage.group_of(cache_layer)]
        pos = self.position
        cos, sin = (pos.cos, pos.sin) if pos else (None, None)
        qk = ctx.rows("mixed_attention.qk", self.q_width + self.k_width)
        q = qk[:, :self.q_width]
        if writes_cache:
            product(ctx, qk, hn, self.w_qk, self.w_qk_tiles)
            k = qk[:, self.q_width:]
        else:       # this run of the layer reads the keys that another run wrote
            ops.linear(q, hn, self.w_qk[:self.q_width])
            k = None
        ops.attention_mix_prepare(q, k, ctx.positions, ctx.token_segment, tables, cos, sin, cache, H, G, D, ctx.page_size,
                                  ctx.max_position, norm=self.qk_norm is not None, eps=self.norm_eps)
        att = ctx.rows("mixed_attention.out", self.q_width)
        sink = "zero" if self.sink == "zero" else self.sinks
        if self.matrix:
            items = ctx.extra[self.items_key]
            # the most key tiles an item can have: a chunk's, or the context's (under a captured graph the block
            # table's whole width, so that a replay runs what was recorded)
            span = self.chunk or ctx.host.get("graph.max_context", ctx.max_position + 1)
            count = items.shape[0]
            splits = max(1, min(-(-span // 16) // 4, _WORKGROUPS_WANTED // count, _MOST_SPLITS))
            while splits > 1 and ops.attention_mix_partial_words(count, H, D, splits) > _PARTIAL_LIMIT:
                splits -= 1
            partial = None
            if splits > 1:
                partial = ctx.workspace.flat("mixed_attention.partial", ops.attention_mix_partial_words(count, H, D, splits),
                                             torch.float32)
            ops.attention_mix_bf16(att, q, cache, items, tables, H, G, D, ctx.page_size, self.scale, mix_t=self.mix_t,
                                   chunk=self.chunk, sink=sink, splits=splits, partial=partial)
        else:
            ops.attention_mix(att, q, cache, ctx.positions, ctx.token_segment, tables, H, G, D, ctx.page_size, self.scale,
                              mix=self.mix, chunk=self.chunk, sink=sink)
        product(ctx, x, att, self.w_o, self.w_o_tiles, add=True)
