"""Rotary position encoding, half-split pairing (j, j + d/2).

f_j = theta^(-2j/d), angle = position * f_j; the rotation itself is fused into
the kernel that follows the q/k/v product (reference: RopeKernel,
src/backends/cuda/ops/layers.cu:80-115; ops/layers.h:35-58).  The frequencies
are computed once in float64 and rounded to float32; the angle and its cosine
and sine are float32, once per step for all layers.

Interface of a position encoding: `prepare(ctx)` returns a float32 table
[T, rotary_dim/2, 2] of (cos, sin) for this step's tokens, or None for no
rotation.  An encoding that rotates only a part of each head says so with its
attributes `rotary_dim` (how many elements) and `begin` (the first of them;
0 if absent): the elements outside pass through (the reference's own partial
rotation takes the trailing part of a head, src/backends/cuda/ops/mla.cu:24-46).

`scaling` stretches the encoding for longer contexts than it was trained on.  {"factor": s}: every frequency is
divided by s.  {"factor": s, "original": L, "fast": b, "slow": a}: the frequencies are blended by a ramp over their
index i,

    at(t) = d ln(L / (2 pi t)) / (2 ln theta)        the index whose wave makes t turns over L positions
    lo = max(floor(at(b)), 0),  hi = min(ceil(at(a)), d - 1),  r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1)
    f_i' = f_i / s * r_i + f_i (1 - r_i)

(fast waves stay, slow ones are stretched), and cosine and sine are both multiplied by `gain` = 0.1 ln(s) + 1.
Which elements of a head a table's pair j turns is the business of the kernel that applies it.
"""
from __future__ import annotations

import math
from typing import Any, Dict, Optional

import torch

from .. import ops
from .base import PositionEncoding, register_part


class Rotary(PositionEncoding):
    graph_safe = True

    def __init__(self, theta: float, rotary_dim: int, begin: int = 0, scaling: Optional[Dict[str, Any]] = None):
        if rotary_dim <= 0 or rotary_dim % 2:
            raise ValueError(f"rotary_dim {rotary_dim} must be positive and even")
        if theta <= 0:
            raise ValueError("theta must be positive")
        if begin < 0:
            raise ValueError("the rotated part cannot begin before the head")
        self.theta, self.rotary_dim, self.begin = float(theta), int(rotary_dim), int(begin)
        self.scaling = dict(scaling) if scaling else None
        self.gain = 1.0
        if self.scaling is not None:
            extra = set(self.scaling) - {"factor", "original", "fast", "slow"}
            ramp = [k for k in ("original", "fast", "slow") if k in self.scaling]
            if extra or "factor" not in self.scaling or len(ramp) not in (0, 3):
                raise ValueError(f"scaling {self.scaling!r}: a factor alone, or factor, original, fast and slow")
            if float(self.scaling["factor"]) <= 0 or any(float(self.scaling[k]) <= 0 for k in ramp):
                raise ValueError("the numbers of a scaling must be positive")
            if ramp:
                if self.theta == 1.0:
                    raise ValueError("a ramp over the frequencies needs a theta other than 1")
                self.gain = 0.1 * math.log(float(self.scaling["factor"])) + 1.0
        self.inv_freq = None

    def frequencies(self) -> torch.Tensor:
        d = self.rotary_dim
        j = torch.arange(d // 2, dtype=torch.float64)
        f = torch.pow(torch.tensor(self.theta, dtype=torch.float64), -2.0 * j / d)
        sc = self.scaling
        if sc is not None:
            factor = float(sc["factor"])
            if "original" in sc:
                at = lambda turns: d * math.log(float(sc["original"]) / (2.0 * math.pi * float(turns))) / (2.0 * math.log(self.theta))
                lo, hi = max(math.floor(at(sc["fast"])), 0), min(math.ceil(at(sc["slow"])), d - 1)
                ramp = torch.clamp((j - lo) / max(hi - lo, 0.001), 0.0, 1.0)
                f = f / factor * ramp + f * (1.0 - ramp)
            else:
                f = f / factor
        return f.to(torch.float32)

    def bind(self, tensors, rt) -> None:
        self.inv_freq = self.frequencies().to(rt.device)

    def prepare(self, ctx):
        key = ("rope", self.theta, self.rotary_dim, tuple(sorted(self.scaling.items())) if self.scaling else None)
        table = ctx.memo.get(key)
        if table is None:
            table = ctx.rt.empty((ctx.num_tokens, self.rotary_dim // 2, 2), torch.float32)
            ops.rope_table(table, ctx.positions, self.inv_freq, self.gain)
            ctx.memo[key] = table
        return table


register_part("position", "rope", Rotary)
