"""A feed-forward of many small gated experts, of which every token uses `top`.

"table_moe": no router.  A table [vocabulary, top] of integers gives every token id its experts (the
entries of a row differ); each counts 1 / top.  Expert: down(act(gate(h)) * up(h)), act the SiLU, no
biases; the output is the weighted sum of the chosen experts' outputs, added to the residual stream in
float32.  The experts' matrices are stacked [experts, rows, columns] when they are bound; the lookup
runs on the device from the step's token ids, so a step may be replayed from a recorded graph.  A step
with more (token, expert) pairs than experts groups the pairs by expert on the device and multiplies them
in tiles on the matrix cores (bfloat16, sizes that are multiples of 32); a step of few tokens, and
float32, reads each token's experts row by row.
"""
from __future__ import annotations

import torch

from ..config.specs import FeedForwardSpec
from ..kernels import ops
from ..weights.spec import TensorSpec
from .base import FeedForward, LazyNorm, register_feed_forward


@register_feed_forward("table_moe")
class TableMoE(FeedForward):
    graph_safe = True

    def __init__(self, spec: FeedForwardSpec, prefix: str, dtype: torch.dtype):
        self.prefix, self.dtype = prefix, dtype
        self.hidden = spec.get("hidden")
        self.intermediate = spec.get("intermediate")
        self.experts, self.top = spec.get("experts"), spec.get("top")
        self.vocab = spec.get("vocab")
        if spec.get("activation", "silu") != "silu":
            raise ValueError("the experts' activation is the SiLU")
        if not 1 <= self.top <= self.experts:
            raise ValueError(f"a token uses 1 to {self.experts} experts, not {self.top}")
        given = dict(spec.get("names") or ())
        self.expert_names = given.get("expert", "experts.{}.")           # a format for the expert's number
        self.roles = {r: given.get(r, d) for r, d in dict(gate="gate_proj.weight", up="up_proj.weight",
                                                         down="down_proj.weight", table="table").items()}

    def _name(self, e: int, role: str) -> str:
        return self.prefix + self.expert_names.format(e) + self.roles[role]

    def tensor_specs(self):
        specs = []
        for e in range(self.experts):
            specs += [TensorSpec(self._name(e, "gate"), (self.intermediate, self.hidden)),
                      TensorSpec(self._name(e, "up"), (self.intermediate, self.hidden)),
                      TensorSpec(self._name(e, "down"), (self.hidden, self.intermediate))]
        specs.append(TensorSpec(self.prefix + self.roles["table"], (self.vocab, self.top), role="table",
                                init=("distinct_in_row", self.experts)))
        return specs

    def bind(self, tensors):
        E = range(self.experts)
        self.w_gate = torch.stack([tensors.pop(self._name(e, "gate")) for e in E]).contiguous()
        self.w_up = torch.stack([tensors.pop(self._name(e, "up")) for e in E]).contiguous()
        self.w_down = torch.stack([tensors.pop(self._name(e, "down")) for e in E]).contiguous()
        self.table = tensors.pop(self.prefix + self.roles["table"]).contiguous()
        lo, hi = int(self.table.min()), int(self.table.max())
        if lo < 0 or hi >= self.experts:
            raise ValueError(f"{self.prefix + self.roles['table']} names experts {lo}..{hi}, the layer has {self.experts}")

    def forward_add(self, ctx, x, h):
        hn = h.tensor() if isinstance(h, LazyNorm) else h
        n, top = ctx.n, self.top
        # more pairs than experts: grouped by expert, an expert's matrices are read once for all its tokens
        if n * top > self.experts and ops.moe_grouped_fits(self.dtype, self.hidden, self.intermediate) \
                and hn.data_ptr() % 16 == 0 and hn.stride(0) % 8 == 0:
            ws = ctx.workspace
            order = ws.flat("table_moe.order", ws.capacity * top, torch.int32)
            tiles = ws.flat("table_moe.tiles", 3 * ops.moe_group_tiles(ws.capacity, top, self.experts) + 1, torch.int32)
            act = ctx.rows("table_moe.act", top * self.intermediate)
            y = ctx.rows("table_moe.rows", top * self.hidden, torch.float32) if top > 1 else None
            ops.moe_grouped(x, hn, self.w_gate, self.w_up, self.w_down, top, order, tiles, act, y, weight=1.0 / top,
                            table=self.table, token_ids=ctx.token_ids)
            return
        act = ctx.rows("table_moe.act", self.top * self.intermediate).view(ctx.n * self.top, self.intermediate)
        ops.moe_up(act, hn, self.w_gate, self.w_up, self.top, table=self.table, token_ids=ctx.token_ids)
        ops.moe_down(x, act, self.w_down, self.top, weight=1.0 / self.top, table=self.table, token_ids=ctx.token_ids)
