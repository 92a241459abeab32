"""The gated feed-forward (/root/reference/internal/llm/forward.go:110-114,
/root/reference/internal/ggml/ops.go:159-165): down(activation(gate(h)) * up(h)), added to
the residual stream; the reference's activation is the SiLU, and which one it is is a
parameter of the part (`activation`: one of `ops.GATE_ACTIVATIONS`).  gate and up run as
one product over a weight whose rows alternate gate_j, up_j, so that the gate is the
product's epilogue (and a step of at most 64 tokens folds the norm in front of it into
the same launch).

"dense_mlp" is the feed-forward without a gate: down(activation(up(h) + b_up)) + b_down, the
activation one of `ops.ROW_ACTIVATIONS` ("relu2": the square of relu; "xielu": with two learned numbers
p, q of a tensor, softplus(p) z^2 + z / 2 above zero and (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2 at
and below it), the biases optional.  It
writes float32 rows (`forward_into`) and leaves the last bias to whoever adds the rows to the
residual stream (`output_bias`): a block that norms them first folds it into that launch."""
from __future__ import annotations

import torch

from ..config.specs import FeedForwardSpec
from ..kernels import ops
from ..weights.spec import TensorSpec
from .base import FeedForward, LazyNorm, register_feed_forward


@register_feed_forward("gated_mlp")
class GatedMLP(FeedForward):
    graph_safe = True
    takes_lazy_norm = True
    emits_norm = True
    second_half_rows = ops.SKINNY_MAX_ROWS

    def __init__(self, spec: FeedForwardSpec, prefix: str, dtype: torch.dtype):
        self.hidden = spec.get("hidden")
        self.intermediate = spec.get("intermediate")
        self.activation = spec.get("activation", "silu")
        if self.activation not in ops.GATE_ACTIVATIONS:
            raise ValueError(f"the gated feed-forward has the activations {sorted(ops.GATE_ACTIVATIONS)}, "
                             f"not {self.activation!r}")
        self.prefix, self.dtype = prefix, dtype
        self.w_gate_up = self.w_down = None

    def tensor_specs(self):
        p = self.prefix
        return [TensorSpec(p + "gate_proj.weight", (self.intermediate, self.hidden)),
                TensorSpec(p + "up_proj.weight", (self.intermediate, self.hidden)),
                TensorSpec(p + "down_proj.weight", (self.hidden, self.intermediate))]

    def bind(self, tensors):
        p = self.prefix
        self.w_gate_up = torch.stack([tensors.pop(p + "gate_proj.weight"), tensors.pop(p + "up_proj.weight")],
                                     dim=1).reshape(2 * self.intermediate, self.hidden).contiguous()
        self.w_down = tensors.pop(p + "down_proj.weight").contiguous()
        # a second copy in tiles for steps of up to 64 rows, whose products stream the weights
        self.aligned = self.dtype == torch.bfloat16 and self.hidden % 8 == 0 and self.intermediate % 8 == 0
        tiles = ops.tile_weights_if_room(self.w_gate_up, self.w_down) if self.aligned else None
        self.streams = tiles is not None
        self.w_gate_up_tiles, self.w_down_tiles = tiles if tiles else (None, None)
        if not self.streams:      # (nobody finishes a norm here that the part before has begun)
            self.second_half_rows = 0

    def forward_add(self, ctx, x, h, then=None):
        F, n = self.intermediate, ctx.n
        act = ctx.rows("mlp.act", F)
        aligned = self.aligned
        lazy = isinstance(h, LazyNorm)
        if self.streams and n <= ops.SKINNY_MAX_ROWS:        # both products stream the weights' tiles
            w = self.w_gate_up_tiles
            halves = h.row_scale() if lazy else None     # (offered for few rows only)
            norm = None
            if halves is None and lazy and n <= ops.FUSED_NORM_MAX_ROWS and ops.norm_fusion_pays(*w.shape):
                norm = h.fusable()
            # the gate as the product's epilogue, where it is the reference's; another activation is a
            # kernel of its own over the product's alternating columns (the kernels for few rows have
            # no register to spare for a choice in their loops)
            silu = self.activation == "silu"
            out, epilogue = (act, "swiglu") if silu else (ctx.rows("mlp.gate_up", 2 * F), "bf16")
            if halves:        # the norm's first half came with the product before; both projections and the gate
                ops.linear_fused(out, halves[0], w, epilogue, row_scale=halves[1], **ctx.workspace.product_scratch(n, w))
            elif norm:        # norm, both projections and the gate in one launch
                ops.linear_fused(out, h.x, w, epilogue, norm_weight=norm[0], eps=norm[1])
            else:
                ops.linear_fused(out, h.tensor() if lazy else h, w, epilogue, **ctx.workspace.product_scratch(n, w))
            if not silu:
                ops.swiglu(act, out[:, 0::2], out[:, 1::2], activation=self.activation)
            # the down projection adds into x and, if asked, begins the norm that follows
            emit = then.offer() if then is not None else None
            ops.linear_fused(x, act, self.w_down_tiles, "add", emit=emit,
                             **ctx.workspace.product_scratch(n, self.w_down_tiles))
            return
        hn = h.tensor() if lazy else h
        if aligned:   # the gate in the product's epilogue
            ops.linear(act, hn, self.w_gate_up, gate=True, activation=self.activation)
        else:
            gate_up = ctx.rows("mlp.gate_up", 2 * F)
            ops.linear(gate_up, hn, self.w_gate_up)
            ops.swiglu(act, gate_up[:, 0::2], gate_up[:, 1::2], activation=self.activation)
        # the down projection adds into x and, if asked, goes on with the norm that follows
        # (where its K is cut over workgroups: the kernel that adds the cuts up has the row at hand)
        cut = ctx.workspace.split_scratch(n, self.w_down)
        after = then.offer_whole() if then is not None and aligned and cut else None
        if after:
            ops.linear_add_norm(x, act, self.w_down, after["out"], after["weight"], after["eps"], **cut)
        else:
            ops.linear(x, act, self.w_down, accumulate=True, **cut)


@register_feed_forward("dense_mlp")
class DenseMLP(FeedForward):
    graph_safe = True

    def __init__(self, spec: FeedForwardSpec, prefix: str, dtype: torch.dtype):
        self.hidden = spec.get("hidden")
        self.intermediate = spec.get("intermediate")
        self.activation = spec.get("activation", "relu2")
        self.has_bias = bool(spec.get("bias", False))
        if self.activation not in ops.ROW_ACTIVATIONS:
            raise ValueError(f"the dense feed-forward has the activations {sorted(ops.ROW_ACTIVATIONS)}, "
                             f"not {self.activation!r}")
        self.prefix, self.dtype = prefix, dtype
        given = dict(spec.get("names") or ())
        defaults = dict(up="up_proj.weight", up_bias="up_proj.bias", down="down_proj.weight", down_bias="down_proj.bias",
                        activation="act_fn")
        self.names = {role: prefix + given.get(role, default) for role, default in defaults.items()}
        self.output_bias = None          # float32; added by whoever takes the rows of forward_into

    def tensor_specs(self):
        n = self.names
        specs = [TensorSpec(n["up"], (self.intermediate, self.hidden)), TensorSpec(n["down"], (self.hidden, self.intermediate))]
        if self.has_bias:
            specs += [TensorSpec(n["up_bias"], (self.intermediate,), role="vector"),
                      TensorSpec(n["down_bias"], (self.hidden,), role="vector")]
        if self.activation == "xielu":
            specs.append(TensorSpec(n["activation"], (2,), role="vector"))
        return specs

    def bind(self, tensors):
        n = self.names
        self.w_up, self.w_down = tensors.pop(n["up"]).contiguous(), tensors.pop(n["down"]).contiguous()
        self.up_bias = tensors.pop(n["up_bias"]).to(self.dtype).contiguous() if self.has_bias else None
        self.output_bias = tensors.pop(n["down_bias"]).to(torch.float32).contiguous() if self.has_bias else None
        self.numbers = (0.0, 0.0)
        if self.activation == "xielu":      # (two numbers, read once: the kernels take them as arguments)
            p, q = torch.nn.functional.softplus(tensors.pop(n["activation"]).to(torch.float64).cpu()).tolist()
            self.numbers = (p, 0.5 + q)
        # a second copy in tiles for steps of up to 64 rows, whose products stream the weights
        self.w_up_tiles = self.w_down_tiles = None
        if self.dtype == torch.bfloat16 and self.hidden % 8 == 0 and self.intermediate % 8 == 0:
            self.w_up_tiles, self.w_down_tiles = ops.tile_weights_if_room(self.w_up, self.w_down) or (None, None)

    def _product(self, ctx, out, x, weight, tiles):
        n = x.shape[0]
        if tiles is not None and n <= ops.SKINNY_MAX_ROWS:
            ops.linear_fused(out, x, tiles, "f32" if out.dtype == torch.float32 else "bf16",
                             **ctx.workspace.product_scratch(n, tiles))
        else:
            ops.linear(out, x, weight, **ctx.workspace.split_scratch(n, weight))

    def forward_into(self, ctx, out, h):
        """out (float32 [n, hidden]) = down(activation(up(h) + b_up)); `output_bias` is not added."""
        hn = h.tensor() if isinstance(h, LazyNorm) else h
        act = ctx.rows("dense_mlp.act", self.intermediate)
        self._product(ctx, act, hn, self.w_up, self.w_up_tiles)
        ops.bias_act(act, act, self.up_bias, self.activation, self.numbers)
        self._product(ctx, out, act, self.w_down, self.w_down_tiles)

    def forward_add(self, ctx, x, h):
        if self.output_bias is None:        # the down product adds straight into the stream
            hn = h.tensor() if isinstance(h, LazyNorm) else h
            act = ctx.rows("dense_mlp.act", self.intermediate)
            self._product(ctx, act, hn, self.w_up, self.w_up_tiles)
            ops.bias_act(act, act, self.up_bias, self.activation, self.numbers)
            n = act.shape[0]
            if self.w_down_tiles is not None and n <= ops.SKINNY_MAX_ROWS:
                ops.linear_fused(x, act, self.w_down_tiles, "add", **ctx.workspace.product_scratch(n, self.w_down_tiles))
            else:
                ops.linear(x, act, self.w_down, accumulate=True, **ctx.workspace.split_scratch(n, self.w_down))
            return
        y = ctx.rows("mixer.rows_out", self.hidden, torch.float32)
        self.forward_into(ctx, y, h)
        if self.output_bias is not None:
            ops.bias_act(y, y, self.output_bias, "none")
        ops.residual_add(x, y)
