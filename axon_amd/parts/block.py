"""The arrangement of a layer's parts around the residual stream.

"prenorm": x += mixer(norm1(x)); x += feed_forward(norm2(x)), the order of
src/model.rs:2980-3055.  The residual stream `x` is float32 and is updated in place: the
mixer and the feed-forward add their output to it in the epilogue of their last product.
"""
from __future__ import annotations

from typing import List

import torch

from ..config.base import ConfigError
from .base import ROUNDED_STREAM, Block, CacheBinding, TensorDecl, register_block

# A norm behind a product whose kernel holds the finished rows anyway can be written by that
# kernel, and a norm before a product of few rows can be worked out inside that product (the same
# bits as the norm's own pass, both): the block asks its parts, step by step.


class PreNormBlock(Block):
    graph_safe = True
    norm1_name = "input_layernorm.weight"
    norm2_name = "post_attention_layernorm.weight"

    def __init__(self, norm_factory, mixer, feed_forward, prefix):
        super().__init__(norm_factory, mixer, feed_forward, prefix)
        self.norm1 = norm_factory(self.norm1_name)
        self.norm2 = norm_factory(self.norm2_name)

    def tensors(self) -> List[TensorDecl]:
        return self.norm1.tensors() + self.mixer.tensors() + self.norm2.tensors() + self.feed_forward.tensors()

    def load(self, store, rt) -> None:
        for part in (self.norm1, self.mixer, self.norm2, self.feed_forward):
            part.load(store, rt)

    def first_norm(self):
        return self.norm1

    def last_part(self):
        return self.feed_forward

    def forward(self, ctx, binding: CacheBinding, x, normed=None, following=None) -> None:
        h = normed
        if h is None:
            h = self.preceding_of(ctx, self.norm1, self.mixer, x)
        if h is None:
            h = self.norm1.forward(ctx, x)
        second = self.following_of(ctx, self.mixer, self.norm2, x.shape[0])
        if second is not None:
            self.mixer.forward(ctx, binding, h, x, second)
            h = second.values
        else:
            self.mixer.forward(ctx, binding, h, x)
            h = self.preceding_of(ctx, self.norm2, self.feed_forward, x)
            if h is None:
                h = self.norm2.forward(ctx, x)
        if following is not None:
            self.feed_forward.forward(ctx, h, x, following)
        else:
            self.feed_forward.forward(ctx, h, x)


class ShortNamedPreNormBlock(PreNormBlock):
    """The same arrangement for checkpoints that call the norms `norm1` and `norm2`; a layer may have no
    feed-forward (it then has no second norm either)."""
    norm1_name = "norm1"
    norm2_name = "norm2"

    def __init__(self, norm_factory, mixer, feed_forward, prefix):
        Block.__init__(self, norm_factory, mixer, feed_forward, prefix)
        self.norm1 = norm_factory(self.norm1_name)
        self.norm2 = norm_factory(self.norm2_name) if feed_forward is not None else None

    def parts(self):
        return [p for p in (self.norm1, self.mixer, self.norm2, self.feed_forward) if p is not None]

    def tensors(self) -> List[TensorDecl]:
        return [d for p in self.parts() for d in p.tensors()]

    def load(self, store, rt) -> None:
        for part in self.parts():
            part.load(store, rt)

    def last_part(self):
        return self.feed_forward if self.feed_forward is not None else self.mixer

    def forward(self, ctx, binding: CacheBinding, x, normed=None, following=None) -> None:
        if self.feed_forward is not None:
            return super().forward(ctx, binding, x, normed, following)
        h = normed
        if h is None:
            h = self.preceding_of(ctx, self.norm1, self.mixer, x)
        if h is None:
            h = self.norm1.forward(ctx, x)
        if following is not None:
            self.mixer.forward(ctx, binding, h, x, following)
        else:
            self.mixer.forward(ctx, binding, h, x)


class SublayerNormBlock(Block):
    """x += mult * norm1(mixer(x)); x += mult * norm2(feed_forward(x)): the norms sit on the sublayers'
    outputs, the sublayers read the residual stream itself (rounded to the compute dtype for their
    products), and a layer may have no feed-forward.  The norm, the scaling and the sum are one
    32-bit pass over the sublayer's 32-bit output, which also leaves the new rows rounded for the
    next sublayer.  The norms are RMS norms (they hand over a gain and an eps).  `residual_mult`
    comes with the norm's parameters."""
    graph_safe = True
    norm1_name = "norm1"
    norm2_name = "norm2"

    def __init__(self, norm_factory, mixer, feed_forward, prefix):
        super().__init__(norm_factory, mixer, feed_forward, prefix)
        self.norm1 = norm_factory(self.norm1_name)
        self.norm2 = norm_factory(self.norm2_name) if feed_forward is not None else None
        for norm in (self.norm1, self.norm2):
            if norm is not None and not (hasattr(norm, "gain") and hasattr(norm, "eps")):
                raise ConfigError("a norm on a sublayer's output is an RMS norm (a gain and an eps)")
        self.mult = float(self.norm1.params.get("residual_mult", 1.0))

    def parts(self):
        return [p for p in (self.norm1, self.mixer, self.norm2, self.feed_forward) if p is not None]

    def tensors(self) -> List[TensorDecl]:
        return [d for p in self.parts() for d in p.tensors()]

    def load(self, store, rt) -> None:
        for part in self.parts():
            part.load(store, rt)

    @staticmethod
    def _run(part, ctx, y, *args) -> None:
        """y = part(...): stored by the part's last product where it can, else added into zeros."""
        if getattr(part, "stores_output", False):
            part.forward(ctx, *args, y, accumulate=False)
        else:
            ctx.rt.k.fill_f32(y.view(-1), 0.0)
            part.forward(ctx, *args, y)

    def forward(self, ctx, binding: CacheBinding, x, normed=None, following=None) -> None:
        k, rt = ctx.rt.k, ctx.rt
        exact = rt.dtype == torch.float32            # the 32-bit path: the sublayers read x as it is
        h = x if exact else k.round_rows(x, ctx.ws.take(tuple(x.shape), rt.dtype))
        y = ctx.ws.take(tuple(x.shape), torch.float32)
        self._run(self.mixer, ctx, y, binding, h)
        if self.feed_forward is None:
            k.norm_add(y, self.norm1.gain, self.norm1.eps, self.mult, x)
            return
        h = x if exact else ctx.ws.take(tuple(x.shape), rt.dtype)
        k.norm_add(y, self.norm1.gain, self.norm1.eps, self.mult, x, None if exact else h)
        self._run(self.feed_forward, ctx, y, h)
        k.norm_add(y, self.norm2.gain, self.norm2.eps, self.mult, x)


class PostNormBlock(Block):
    """x <- norm1(alpha x + mixer(x)); x <- norm2(alpha x + feed_forward(x)): the norms sit behind the
    sums, the sublayers read the stream itself (rounded to the compute dtype for their products), and
    a layer may have no feed-forward (it then has no second norm).  The scaling, the sum and the norm
    are one 32-bit pass over the sublayer's 32-bit output, which also leaves the new rows rounded for
    the next sublayer, the next block's too.  The norms are RMS or layer norms (a gain, an eps and a
    `kind`); `stream_alpha` comes with the norm's parameters."""
    graph_safe = True
    norm1_name = "norm1"
    norm2_name = "norm2"

    def __init__(self, norm_factory, mixer, feed_forward, prefix):
        super().__init__(norm_factory, mixer, feed_forward, prefix)
        self.norm1 = norm_factory(self.norm1_name)
        self.norm2 = norm_factory(self.norm2_name) if feed_forward is not None else None
        for norm in (self.norm1, self.norm2):
            if norm is not None and not all(hasattr(norm, a) for a in ("gain", "eps", "kind")):
                raise ConfigError("a norm behind a sum is an RMS norm or a layer norm (a gain, an eps and a kind)")
        self.alpha = float(self.norm1.params.get("stream_alpha", 1.0))

    def parts(self):
        return [p for p in (self.norm1, self.mixer, self.norm2, self.feed_forward) if p is not None]

    def tensors(self) -> List[TensorDecl]:
        return [d for p in self.parts() for d in p.tensors()]

    def load(self, store, rt) -> None:
        for part in self.parts():
            part.load(store, rt)

    _run = staticmethod(SublayerNormBlock._run)

    def forward(self, ctx, binding: CacheBinding, x, normed=None, following=None) -> None:
        k, rt = ctx.rt.k, ctx.rt
        exact = rt.dtype == torch.float32            # the 32-bit path: the sublayers read x as it is
        h = x
        if not exact:
            left = ctx.shared.get(ROUNDED_STREAM)    # the block before left the rows it wrote, rounded
            h = left[1] if left is not None and left[0] is x else k.round_rows(x, ctx.ws.take(tuple(x.shape), rt.dtype))
        y = ctx.ws.take(tuple(x.shape), torch.float32)
        self._run(self.mixer, ctx, y, binding, h)
        h = None if exact else ctx.ws.take(tuple(x.shape), rt.dtype)
        k.sum_norm(y, self.alpha, self.norm1.gain, self.norm1.eps, self.norm1.kind, x, h)
        if self.feed_forward is not None:
            self._run(self.feed_forward, ctx, y, x if exact else h)
            k.sum_norm(y, self.alpha, self.norm2.gain, self.norm2.eps, self.norm2.kind, x, h)
        ctx.shared[ROUNDED_STREAM] = None if exact else (x, h)


class ParallelBlock(Block):
    """h = norm1(x); x += mixer(h) + feed_forward(h): one norm, and both sublayers read its output (a
    layer may have no feed-forward).  Each sublayer adds into the 32-bit stream in the epilogue of its
    last product."""
    graph_safe = True
    norm1_name = "norm1"

    def __init__(self, norm_factory, mixer, feed_forward, prefix):
        super().__init__(norm_factory, mixer, feed_forward, prefix)
        self.norm1 = norm_factory(self.norm1_name)

    def parts(self):
        return [p for p in (self.norm1, self.mixer, self.feed_forward) if p is not None]

    def tensors(self) -> List[TensorDecl]:
        return [d for p in self.parts() for d in p.tensors()]

    def load(self, store, rt) -> None:
        for part in self.parts():
            part.load(store, rt)

    def first_norm(self):
        return self.norm1

    def forward(self, ctx, binding: CacheBinding, x, normed=None, following=None) -> None:
        h = normed if normed is not None else self.norm1.forward(ctx, x)
        self.mixer.forward(ctx, binding, h, x)
        if self.feed_forward is not None:
            self.feed_forward.forward(ctx, h, x)


register_block("prenorm", PreNormBlock)
register_block("parallel", ParallelBlock)
register_block("prenorm_short_names", ShortNamedPreNormBlock)
register_block("sublayer_norm", SublayerNormBlock)
register_block("postnorm", PostNormBlock)
