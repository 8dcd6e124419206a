"""Dense gated feed-forward: down( silu(gate(x)) * up(x) ); optionally with biases on the three products and the
clamped activation (`limit` > 0: g = min(gate, limit), u = clamp(up, -limit, limit), g sigmoid(1.702 g) (u + 1)).

gate and up are stacked into one [2I, H] matrix, gate rows first (reference:
src/model/qwen2.cc:1413-1434 load, :1042-1048 forward; SiluMulFusedKernel
layers.cu:512-529).
"""
from __future__ import annotations

from typing import List

import torch

from .base import FeedForward, LazyDelta, ParamSpec, register_part


def stack_rows(tensors):
    """Concatenate along dim 0; mixed storage types widen to float32."""
    if len({t.dtype for t in tensors}) > 1:
        tensors = [t.to(torch.float32) for t in tensors]
    return torch.cat(tensors, dim=0).contiguous()


class BiasedDelta(LazyDelta):
    """A branch's result whose bias per column is not added yet: tensor[t, c] + bias[c].  A consumer that sums
    branches takes both as they are; anybody else gets the sum."""

    def __init__(self, tensor, bias):
        self.tensor, self.bias = tensor, bias

    def materialize(self, ctx):
        from .. import ops
        out = self.tensor.clone()
        ops.add_bias(out, self.bias)
        return out


class DenseMlp(FeedForward):
    graph_safe = True

    def __init__(self, hidden_size: int, width: int, init_std: float = 0.02, bias: bool = False, limit: float = 0.0):
        self.hidden_size, self.width, self.init_std = int(hidden_size), int(width), float(init_std)
        self.bias, self.limit = bool(bias), float(limit)
        self.w_gate_up = self.w_down = self.b_gate_up = self.b_down = None

    def param_specs(self) -> List[ParamSpec]:
        H, I, s = self.hidden_size, self.width, self.init_std
        specs = [ParamSpec("gate_proj.weight", (I, H), std=s), ParamSpec("up_proj.weight", (I, H), std=s),
                 ParamSpec("down_proj.weight", (H, I), std=s)]
        if self.bias:
            specs += [ParamSpec("gate_proj.bias", (I,), std=s), ParamSpec("up_proj.bias", (I,), std=s),
                      ParamSpec("down_proj.bias", (H,), std=s)]
        return specs

    def bind(self, tensors, rt) -> None:
        self.w_gate_up = stack_rows([tensors["gate_proj.weight"], tensors["up_proj.weight"]])
        self.w_down = tensors["down_proj.weight"].contiguous()
        if self.bias:
            self.b_gate_up = stack_rows([tensors["gate_proj.bias"], tensors["up_proj.bias"]])
            self.b_down = tensors["down_proj.bias"].contiguous()

    def forward(self, ctx, x):
        """The result without the last product's bias: whoever adds the result to the stream adds `out_bias()` with
        it (`BiasedDelta`), so that the bias costs no pass of its own."""
        rt = ctx.rt
        y = rt.linear(rt.gated_linear(x, self.w_gate_up, self.limit, self.b_gate_up), self.w_down)
        return y if self.b_down is None else BiasedDelta(y, self.b_down)


class PolyNormMlp(FeedForward):
    """A feed-forward without a gate whose activation blends the normalised first three powers of its input:

        z = x . Wup^T;   y = (a N(z) + b N(z^2) + c N(z^3) + e) . Wdown^T,   N(v) = v / sqrt(mean(v^2) + eps)

    with the powers taken element by element and the four numbers a, b, c, e learned (`act`).  The sums of squares
    and the blend are float32."""

    graph_safe = True

    def __init__(self, hidden_size: int, width: int, norm_eps: float = 1e-6, init_std: float = 0.02):
        self.hidden_size, self.width = int(hidden_size), int(width)
        self.norm_eps, self.init_std = float(norm_eps), float(init_std)
        self.w_up = self.w_down = self.coef = None

    def param_specs(self) -> List[ParamSpec]:
        H, I, s = self.hidden_size, self.width, self.init_std
        return [ParamSpec("up_proj.weight", (I, H), std=s), ParamSpec("down_proj.weight", (H, I), std=s),
                ParamSpec("act", (4,), std=0.3, mean=0.3)]

    def bind(self, tensors, rt) -> None:
        self.w_up, self.w_down = tensors["up_proj.weight"].contiguous(), tensors["down_proj.weight"].contiguous()
        self.coef = tensors["act"].to(torch.float32).contiguous()

    def forward(self, ctx, x):
        from .. import ops
        rt = ctx.rt
        z = rt.linear(x, self.w_up)
        y = rt.empty(tuple(z.shape))
        ops.polynorm(z, self.coef, y, self.norm_eps)
        return rt.linear(y, self.w_down)


register_part("feed_forward", "dense_mlp", DenseMlp)
register_part("feed_forward", "polynorm_mlp", PolyNormMlp)
