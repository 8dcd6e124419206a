"""Arrangement of a layer's parts.  `prenorm`:

    h += pending;  a = mixer(norm1(h));  h += a;  f = feed_forward(norm2(h));  pending = f

(reference: src/model/qwen2.cc:908-1051).  The residual stream h is float32 and
is updated inside the norm kernel, so each add is fused with the norm after it;
the last pending delta is added by the model's final norm.  A feed-forward that
says so gets norm2 unapplied (`LazyNorm`) and applies it in its first kernel.
"""
from __future__ import annotations

import torch

from .. import ops
from .base import Block, LazyDelta, LazyNorm, register_part, resolve_delta
from .dense_mlp import BiasedDelta
from .gain_shift import WeightedSum
from .norm import NormedDelta


class PreNormBlock(Block):
    graph_safe = True
    part_kinds = {"mixer": "mixer", "feed_forward": "feed_forward", "mixer_norm": "norm", "feed_forward_norm": "norm"}

    def forward(self, ctx, h, pending, caches):
        x = self.mixer_norm.forward(ctx, h, pending)
        a = self.mixer.forward(ctx, x, caches.get("mixer"))
        if self.feed_forward.takes_lazy_norm:
            return self.feed_forward.forward(ctx, LazyNorm(self.feed_forward_norm, h, a))
        return self.feed_forward.forward(ctx, self.feed_forward_norm.forward(ctx, h, a))


class GainedPreNormBlock(Block):
    """`prenorm` with three optional additions, each a part of its own:

        x = shift(norm1(h + pending));  h += gain1 * mixer(x);  pending = gain2 * feed_forward(norm2(h))

    `mixer_gain` / `feed_forward_gain` (kind "gain"): a learned gain per channel on the branch's result;
    `mixer_shift` (kind "shift"): the mixer reads rows blended with the rows of the tokens before them.  The
    feed-forward and its norm may be left out; the mixer's delta then stays pending for the next layer."""

    graph_safe = True
    part_kinds = {"mixer": "mixer", "feed_forward": "feed_forward", "mixer_norm": "norm", "feed_forward_norm": "norm",
                  "mixer_gain": "gain", "feed_forward_gain": "gain", "mixer_shift": "shift"}
    optional_parts = ("feed_forward", "feed_forward_norm", "mixer_gain", "feed_forward_gain", "mixer_shift")

    def __init__(self, parts):
        super().__init__(parts)
        if (self.feed_forward is None) != (self.feed_forward_norm is None):
            raise KeyError("a feed-forward and the norm before it come together or not at all")

    def forward(self, ctx, h, pending, caches):
        moved = None
        if self.mixer_shift is not None:
            # a norm that shifts in its own kernel leaves the updated stream in a buffer of its own (`moved`)
            x, moved = self.mixer_norm.forward_shifted(ctx, h, pending, self.mixer_shift, caches.get("mixer_shift"))
        else:
            x = self.mixer_norm.forward(ctx, h, pending)
        a = self.mixer.forward(ctx, x, caches.get("mixer"))
        if self.mixer_gain is not None:
            a = self.mixer_gain.apply(resolve_delta(ctx, a))
        if self.feed_forward is None:
            if moved is not None:
                h.copy_(moved)
            return a
        if moved is not None and self.feed_forward_norm.reads_stream_elsewhere:
            # the next norm reads the stream where it is now and writes it back to h
            x = self.feed_forward_norm.forward(ctx, h, a, h_in=moved)
        else:
            if moved is not None:
                h.copy_(moved)
            x = self.feed_forward_norm.forward(ctx, h, a)
        f = self.feed_forward.forward(ctx, x)
        if self.feed_forward_gain is not None:
            f = self.feed_forward_gain.apply(resolve_delta(ctx, f))
        return f


class SandwichNormBlock(Block):
    """A norm before and after each branch:

        h += post1(mixer(norm1(h)));   h += post2(feed_forward(norm2(h)))

    The normalised branch results travel as `NormedDelta`s, so that an RMS norm that follows (the layer's next one,
    the next layer's first, the model's last) forms them, adds them and normalises in one kernel.  The feed-forward
    and its two norms may be left out together."""

    graph_safe = True
    part_kinds = {"mixer": "mixer", "feed_forward": "feed_forward", "mixer_norm": "norm", "mixer_post_norm": "norm",
                  "feed_forward_norm": "norm", "feed_forward_post_norm": "norm"}
    optional_parts = ("feed_forward", "feed_forward_norm", "feed_forward_post_norm")

    def __init__(self, parts):
        super().__init__(parts)
        present = [p is not None for p in (self.feed_forward, self.feed_forward_norm, self.feed_forward_post_norm)]
        if any(present) != all(present):
            raise KeyError("a feed-forward and the norms around it come together or not at all")

    def forward(self, ctx, h, pending, caches):
        x = self.mixer_norm.forward(ctx, h, pending)
        a = NormedDelta(self.mixer.forward(ctx, x, caches.get("mixer")), self.mixer_post_norm)
        if self.feed_forward is None:
            return a
        x = self.feed_forward_norm.forward(ctx, h, a)
        return NormedDelta(self.feed_forward.forward(ctx, x), self.feed_forward_post_norm)


class BranchSum(LazyDelta):
    """The sum of two branches' results, not formed yet: `first` a tensor, `second` a tensor, a `BiasedDelta` or any
    other sum that is not formed (the experts').  Whoever adds it to the stream adds the parts one by one, in
    float32: the first (with a tensor second, and its bias, in the same pass), then what the second knows to fuse
    with the norm that follows."""

    def __init__(self, first, second):
        self.first, self.second = first, second

    def _add_first(self, ctx, h):
        """h += first (+ second where that is a tensor, with its bias); returns what is still to be added."""
        second = self.second
        if isinstance(second, BiasedDelta):
            ops.add_branches(h, self.first, second.tensor, second.bias)
            return None
        if isinstance(second, LazyDelta):
            ops.add_branches(h, self.first)
            return second
        ops.add_branches(h, self.first, second)
        return None

    def materialize(self, ctx):
        total = torch.zeros(tuple(self.first.shape), dtype=torch.float32, device=self.first.device)
        rest = self._add_first(ctx, total)
        if rest is not None:
            ops.add_branches(total, rest.materialize(ctx))
        return total

    def add_rmsnorm(self, ctx, h, weight, eps, rows, out) -> bool:
        """The stream takes the whole sum here, also where only picked rows are normalised (the model's last norm:
        nobody reads the stream after it)."""
        rest = self._add_first(ctx, h)
        if rest is None or not rest.add_rmsnorm(ctx, h, weight, eps, rows, out):
            ops.add_rmsnorm(h, None if rest is None else rest.materialize(ctx), weight, out, eps, rows)
        return True


class ParallelBlock(Block):
    """One norm, and both branches read its result:

        x = norm(h + pending);   pending = mixer(x) + feed_forward(x)

    The feed-forward may be left out.  The sum travels unformed (`BranchSum`) to the next norm."""

    graph_safe = True
    part_kinds = {"norm": "norm", "mixer": "mixer", "feed_forward": "feed_forward"}
    optional_parts = ("feed_forward",)

    def forward(self, ctx, h, pending, caches):
        x = self.norm.forward(ctx, h, pending)
        a = self.mixer.forward(ctx, x, caches.get("mixer"))
        if self.feed_forward is None:
            return a
        return BranchSum(resolve_delta(ctx, a), self.feed_forward.forward(ctx, x))


class PreNormBranchesBlock(Block):
    """`prenorm` whose mixer may have a second mixer beside it, both reading the one norm, each with a constant gain:

        x = norm1(h + pending);  h += ga * mixer(x) + gb * second_mixer(x);  pending = feed_forward(norm2(h))

    `second_mixer`, the gains (kind "gain", parts with a `factor`) and the feed-forward with its norm may be left
    out; without a feed-forward the mixers' result stays pending for the next layer.  Each mixer keeps pages or
    state of its own (`caches` by part name)."""

    graph_safe = True
    part_kinds = {"mixer": "mixer", "second_mixer": "mixer", "mixer_gain": "gain", "second_mixer_gain": "gain",
                  "feed_forward": "feed_forward", "mixer_norm": "norm", "feed_forward_norm": "norm"}
    optional_parts = ("second_mixer", "mixer_gain", "second_mixer_gain", "feed_forward", "feed_forward_norm")

    def __init__(self, parts):
        super().__init__(parts)
        if (self.feed_forward is None) != (self.feed_forward_norm is None):
            raise KeyError("a feed-forward and the norm before it come together or not at all")
        if self.second_mixer is None and self.second_mixer_gain is not None:
            raise KeyError("a gain for a second mixer that is not there")
        for gain in (self.mixer_gain, self.second_mixer_gain):
            if gain is not None and not hasattr(gain, "factor"):
                raise KeyError("the gains of this arrangement are constants (parts with a `factor`)")

    def forward(self, ctx, h, pending, caches):
        x = self.mixer_norm.forward(ctx, h, pending)
        a = self.mixer.forward(ctx, x, caches.get("mixer"))
        fa = 1.0 if self.mixer_gain is None else self.mixer_gain.factor
        if self.second_mixer is not None:
            b = self.second_mixer.forward(ctx, x, caches.get("second_mixer"))
            fb = 1.0 if self.second_mixer_gain is None else self.second_mixer_gain.factor
            a = WeightedSum([(resolve_delta(ctx, a), fa), (resolve_delta(ctx, b), fb)])
        elif fa != 1.0:
            a = WeightedSum([(resolve_delta(ctx, a), fa)])
        if self.feed_forward is None:
            return a
        if self.feed_forward.takes_lazy_norm:
            return self.feed_forward.forward(ctx, LazyNorm(self.feed_forward_norm, h, a))
        return self.feed_forward.forward(ctx, self.feed_forward_norm.forward(ctx, h, a))


register_part("block", "prenorm", PreNormBlock)
register_part("block", "prenorm_branches", PreNormBranchesBlock)
register_part("block", "parallel", ParallelBlock)
register_part("block", "sandwich_norm", SandwichNormBlock)
register_part("block", "prenorm_gained", GainedPreNormBlock)
