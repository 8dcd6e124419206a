"""Two small parts that sit between a layer's branches and its residual stream.

`ChannelGain`: a branch's result times a learned number per channel before it is added (layer scale).  The
product is not formed here: the delta goes on as a `ScaledDelta`, and the norm that adds it applies the gain.

`PreviousTokenShift`: x[t] <- x[t] + (x[t-1] - x[t]) * mix, channel by channel, with x[t-1] the row of the token
before in the same sequence as it was before this replacement, and zeros before a sequence's first token.  The last
row of a step is kept per request (float32) for the request's next step.
"""
from __future__ import annotations

from typing import List

import torch

from .. import ops
from .base import BranchGain, LazyDelta, ParamSpec, ScaledDelta, StateNeed, TokenShift, register_part, resolve_delta


class ChannelGain(BranchGain):
    graph_safe = True

    def __init__(self, width: int):
        self.width = int(width)
        self.weight = None

    def param_specs(self) -> List[ParamSpec]:
        return [ParamSpec("weight", (self.width,), std=0.2, mean=1.0)]

    def bind(self, tensors, rt) -> None:
        self.weight = tensors["weight"].to(torch.float32).contiguous()

    def apply(self, delta):
        if isinstance(delta, ScaledDelta):  # a gain on a gain: one vector does both
            return ScaledDelta(delta.tensor, delta.gain * self.weight)
        return ScaledDelta(delta, self.weight)


class ConstantGain(BranchGain):
    """A branch's result times ONE fixed number (a constant of the configuration, no tensor).  Where two branches
    meet, the arrangement forms fa * a + fb * b in one pass (`WeightedSum`); alone it is a `WeightedSum` of one."""

    graph_safe = True

    def __init__(self, factor: float):
        self.factor = float(factor)

    def apply(self, delta):
        return WeightedSum([(delta, self.factor)])


class WeightedSum(LazyDelta):
    """fa * a + fb * b of one or two branches' results (tensors of the run's type), not formed yet; whoever adds it
    to the stream gets the float32 sum, formed in one pass."""

    def __init__(self, terms):
        if not 1 <= len(terms) <= 2:
            raise ValueError("a weighted sum of one or two branches")
        self.terms = list(terms)

    def materialize(self, ctx):
        (a, fa), (b, fb) = self.terms[0], (self.terms[1] if len(self.terms) == 2 else (None, 0.0))
        out = ctx.rt.empty(tuple(a.shape), torch.float32)
        ops.weighted_sum(a, fa, b, fb, out)
        return out


class PreviousTokenShift(TokenShift):
    graph_safe = True  # the rows before come from the step's device arrays and the state, nothing from the host

    def __init__(self, width: int):
        self.width = int(width)
        self.mix = None

    def param_specs(self) -> List[ParamSpec]:
        return [ParamSpec("weight", (self.width,), std=0.2, mean=0.5)]

    def state_need(self) -> StateNeed:
        return StateNeed((self.width,), "float32")

    def bind(self, tensors, rt) -> None:
        self.mix = tensors["weight"].to(torch.float32).contiguous()

    def operands(self, ctx, cache) -> ops.ShiftOperands:
        """What a kernel that shifts on its own way needs."""
        return ops.ShiftOperands(self.mix, cache.state, ctx.seq_of_token, ctx.q_start, ctx.state_slots, ctx.positions)

    def forward(self, ctx, x, cache):
        x = resolve_delta(ctx, x)
        out = torch.empty_like(x)
        ops.token_shift(x, out, self.operands(ctx, cache))
        return out


register_part("gain", "channel_gain", ChannelGain)
register_part("gain", "constant_gain", ConstantGain)
register_part("shift", "previous_token", PreviousTokenShift)
