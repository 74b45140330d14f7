"""Pre-norm residual block: r = x + mixer(norm_in(x)); y = r + ff(norm_post(r))
(src/model/qwen3.cpp:948-968).  The adds run inside the norm kernels on the
32-bit residual stream; the last add of a block is left to the next norm.  A block
without a feed-forward is the first line alone: the mixer's result is what it leaves."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..weights.spec import TensorSpec

from .base import Block, BuildContext, Carried, FeedForward, Mixer, Norm, Normed, Prenormed, ScaledSum


class PreNormBlock(Block):
    def __init__(self, norm_in: Norm, mixer: Mixer, norm_post: Optional[Norm] = None,
                 feed_forward: Optional[FeedForward] = None):
        if (norm_post is None) != (feed_forward is None):
            raise ValueError("a feed-forward and its norm come together")
        self.norm_in = norm_in
        self.mixer = mixer
        self.norm_post = norm_post
        self.feed_forward = feed_forward

    def _parts(self):
        return tuple(p for p in (self.norm_in, self.mixer, self.norm_post, self.feed_forward) if p is not None)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs: Dict[str, TensorSpec] = {}
        for p in self._parts():
            specs.update(p.tensor_specs())
        return specs

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        for p in self._parts():
            p.bind(weights, ctx)

    def entry_norm(self):
        return self.norm_in if self.mixer.folds_norm else None

    def input_norm(self):
        return self.norm_in

    def forward(self, hidden, delta, step, cache, next_norm=None):
        if isinstance(delta, Carried):  # the block before has added everything into the stream itself
            delta = None
        if isinstance(delta, Prenormed):  # made for norm_in by the block before: the add and the norm are done
            x = delta
        elif isinstance(delta, Normed):  # norm_in's result, made together with the rows of `hidden`
            x = delta.x
        else:
            x = self.norm_in.forward(hidden, delta)
        if self.feed_forward is None:
            return self.mixer.forward(x, step, cache)
        fold = self.norm_post.fold(hidden) if self.mixer.folds_norm and self.feed_forward.folds_norm else None
        if fold is not None:
            x = self.mixer.forward(x, step, cache, fold=fold)
        else:
            x = self.norm_post.forward(hidden, self.mixer.forward(x, step, cache))
        fold = next_norm.fold(hidden) if next_norm is not None and self.feed_forward.folds_norm else None
        if fold is not None:
            return self.feed_forward.forward(x, fold=fold)
        y = self.feed_forward.forward(x)
        if isinstance(y, torch.Tensor) and y.dtype != self.ctx.dtype:
            # a sum that a routed feed-forward has kept in 32-bit enters the stream as it is: the norm's kernel
            # that takes a sum of sublayers takes either type
            return ScaledSum(y, None, 1.0)
        return y


class PostNormBlock(Block):
    """Residual block whose norms sit on the sublayers' OUTPUTS:
        x <- x + norm_mix(mixer(x));  x <- x + norm_ff(ff(x))
    The sublayers read the residual stream itself (its rows in the activation type).  Each
    norm's kernel adds its result into the 32-bit stream and hands the new rows on in the
    activation type, so a block leaves nothing to add: it returns a `Carried`.  A block
    without a feed-forward is the first line alone."""

    def __init__(self, norm_mix: Norm, mixer: Mixer, norm_ff: Optional[Norm] = None,
                 feed_forward: Optional[FeedForward] = None):
        if (norm_ff is None) != (feed_forward is None):
            raise ValueError("a feed-forward and its norm come together")
        self.norm_mix = norm_mix
        self.mixer = mixer
        self.norm_ff = norm_ff
        self.feed_forward = feed_forward

    def _parts(self):
        return tuple(p for p in (self.norm_mix, self.mixer, self.norm_ff, self.feed_forward) if p is not None)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs: Dict[str, TensorSpec] = {}
        for p in self._parts():
            specs.update(p.tensor_specs())
        return specs

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        for p in self._parts():
            p.bind(weights, ctx)

    def forward(self, hidden, delta, step, cache, next_norm=None):
        if isinstance(delta, Carried):
            x = delta.x
        else:
            if delta is not None:  # left by a block of another arrangement
                if isinstance(delta, (Prenormed, Normed)):
                    raise ValueError("a block that norms its sublayers' outputs takes no ready-made norm")
                hidden += (delta.total() if hasattr(delta, "total") else delta).to(hidden.dtype)
            x = self.ctx.ops.cast(hidden, self.ctx.dtype)
        x = self.norm_mix.add_normed(hidden, self.mixer.forward(x, step, cache))
        if self.feed_forward is not None:
            y = self.feed_forward.forward(x)
            extra = None
            if isinstance(y, tuple):  # a feed-forward in two parts whose sum the norm's kernel takes
                y, extra = y
            x = self.norm_ff.add_normed(hidden, y, extra)
        return Carried(x)


class ParallelBlock(Block):
    """Residual block whose sublayers run side by side on ONE norm's result:
        h = norm(x);  x <- x + mult * (mixer(h) + ff(h))
    The sum is left to whoever comes next as a `ScaledSum`: the next norm's kernel adds it into
    the 32-bit stream, times `mult`, and norms in the same launch.  A block without a
    feed-forward adds the mixer's result alone."""

    def __init__(self, norm: Norm, mixer: Mixer, feed_forward: Optional[FeedForward] = None, mult: float = 1.0):
        self.norm = norm
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mult = float(mult)

    def _parts(self):
        return tuple(p for p in (self.norm, self.mixer, self.feed_forward) if p is not None)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs: Dict[str, TensorSpec] = {}
        for p in self._parts():
            specs.update(p.tensor_specs())
        return specs

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        for p in self._parts():
            p.bind(weights, ctx)

    def input_norm(self):
        return self.norm

    def forward(self, hidden, delta, step, cache, next_norm=None):
        if isinstance(delta, Carried):  # the block before has added everything into the stream itself
            delta = None
        if isinstance(delta, Prenormed):
            raise ValueError("a block of side-by-side sublayers takes no folded norm")
        h = delta.x if isinstance(delta, Normed) else self.norm.forward(hidden, delta)
        a = self.mixer.forward(h, step, cache)
        b = self.feed_forward.forward(h) if self.feed_forward is not None else None
        return ScaledSum(a, b, self.mult)


class SandwichBlock(Block):
    """Residual block with a norm before and a norm after each sublayer:
        x <- x + norm_mix_out(mixer(norm_in(x)));  x <- x + norm_ff_out(ff(norm_ff_in(x)))
    The norm after a sublayer is applied by a kernel that also adds its result into the 32-bit
    stream, and where the norms have a kernel for it, that launch norms the new rows for whoever
    reads them next (`Norm.add_normed(..., then=)`): the feed-forward's norm, the next block's first
    norm (`next_norm`; the block then returns a `Normed`), so every sublayer costs one norm launch.
    A sublayer may hand its result on as a pair whose sum is meant (two mixers side by side, a routed
    feed-forward with a shared expert): the norm's kernel adds the two.  A block without a feed-forward
    is the first line alone."""

    def __init__(self, norm_in: Norm, mixer: Mixer, norm_mix_out: Norm, norm_ff_in: Optional[Norm] = None,
                 feed_forward: Optional[FeedForward] = None, norm_ff_out: Optional[Norm] = None):
        if not ((norm_ff_in is None) == (feed_forward is None) == (norm_ff_out is None)):
            raise ValueError("a feed-forward and its two norms come together")
        self.norm_in, self.mixer, self.norm_mix_out = norm_in, mixer, norm_mix_out
        self.norm_ff_in, self.feed_forward, self.norm_ff_out = norm_ff_in, feed_forward, norm_ff_out

    def _parts(self):
        return tuple(p for p in (self.norm_in, self.mixer, self.norm_mix_out, self.norm_ff_in, self.feed_forward,
                                 self.norm_ff_out) if p is not None)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs: Dict[str, TensorSpec] = {}
        for p in self._parts():
            specs.update(p.tensor_specs())
        return specs

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        for p in self._parts():
            p.bind(weights, ctx)

    def input_norm(self):
        return self.norm_in

    def chained_norm(self):
        return self.norm_in

    @staticmethod
    def _pair(y):
        return y if isinstance(y, tuple) else (y, None)

    def forward(self, hidden, delta, step, cache, next_norm=None):
        if isinstance(delta, Carried):  # the block before has added everything into the stream itself
            delta = None
        if isinstance(delta, Prenormed):
            raise ValueError("a block with norms on both sides of its sublayers takes no folded norm")
        x = delta.x if isinstance(delta, Normed) else self.norm_in.forward(hidden, delta)
        y, extra = self._pair(self.mixer.forward(x, step, cache))
        if self.feed_forward is None:
            if next_norm is None:
                self.norm_mix_out.add_normed(hidden, y, extra)
                return None
            return Normed(self.norm_mix_out.add_normed(hidden, y, extra, then=next_norm))
        x = self.norm_mix_out.add_normed(hidden, y, extra, then=self.norm_ff_in)
        y, extra = self._pair(self.feed_forward.forward(x))
        if next_norm is None:
            self.norm_ff_out.add_normed(hidden, y, extra)
            return None
        return Normed(self.norm_ff_out.add_normed(hidden, y, extra, then=next_norm))
