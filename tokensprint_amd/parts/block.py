"""Arrangements of a layer's parts around the residual stream.

Pre-norm arrangement: x = x + mixer(norm(x)); x = x + ffn(norm(x))
(engine/nn/layers.py:111-121).  Each residual add is fused into the following norm.
A layer may leave out one of the two sub-layers (its part and its norm together)."""

from __future__ import annotations

import torch

from tokensprint_amd.kernels.stream import NormAhead, NormedRows, fused_rmsnorm_of
from tokensprint_amd.parts.base import (BLOCKS, FEED_FORWARDS, FILTERS, MIXERS, NORMS, Block,
                                        StreamFilter, TensorDecl, SlotStateNeed, register)


@register(BLOCKS, "pre_norm")
class PreNormBlock(Block):
    ROLES = {"mixer_norm": (NORMS, False), "mixer": (MIXERS, False),
             "ffn_norm": (NORMS, False), "feed_forward": (FEED_FORWARDS, False)}

    def __init__(self, parts, ctx):
        super().__init__(parts, ctx)
        if (self.mixer is None) != (self.mixer_norm is None) or \
                (self.feed_forward is None) != (self.ffn_norm is None):
            raise ValueError("pre_norm: a sub-layer and its norm come together")
        if self.mixer is None and self.feed_forward is None:
            raise ValueError("pre_norm: a layer needs a mixer or a feed-forward")

    def entry_hint(self):
        if self.mixer is not None:
            return self.mixer.stream_hint(self.mixer_norm)
        return self.feed_forward.stream_hint(self.ffn_norm)

    def forward(self, resid, delta, batch, cache, write_cache, next_hint=None):
        if self.mixer is not None:
            hint = self.feed_forward.stream_hint(self.ffn_norm) \
                if self.feed_forward is not None else next_hint
            delta, resid = self.mixer.forward_from_stream(
                resid, delta, self.mixer_norm, batch, cache, write_cache, hint=hint)
        if self.feed_forward is not None:
            delta, resid = self.feed_forward.forward_from_stream(
                resid, delta, self.ffn_norm, batch, hint=next_hint)
        return resid, delta


@register(BLOCKS, "sandwich_norm")
class SandwichNormBlock(Block):
    """A norm before and one after each sub-layer:
    x = x + post1(mixer(filter(norm1(x)))); x = x + post2(ffn(norm2(x))).
    The filter (what the mixer reads passes through it, e.g. a token shift) and the
    feed-forward with its two norms may be left out.  With RMS norms the add of the mixer's
    normalised output and the norm in front of the feed-forward are one kernel, and so are
    the norm in front of the mixer and the filter; the stream leaves the block summed up
    (no delta is handed on)."""

    ROLES = {"mixer_norm": (NORMS, True), "mixer_filter": (FILTERS, False),
             "mixer": (MIXERS, True), "mixer_post_norm": (NORMS, True),
             "ffn_norm": (NORMS, False), "feed_forward": (FEED_FORWARDS, False),
             "ffn_post_norm": (NORMS, False)}

    def __init__(self, parts, ctx):
        super().__init__(parts, ctx)
        ffn = (self.ffn_norm, self.feed_forward, self.ffn_post_norm)
        if any(p is None for p in ffn) and any(p is not None for p in ffn):
            raise ValueError("sandwich_norm: a feed-forward comes with both of its norms")

    def _post_add(self, resid, out, post, then=None):
        """resid += post(out); then, if given, the norm `then` of the sum."""
        ops = self.ctx.ops
        fused = fused_rmsnorm_of(post)
        nxt = fused_rmsnorm_of(then) if then is not None else None
        if fused is not None and (then is None or nxt is not None):
            if then is None:
                ops.postnorm_add(resid, out, fused[0], fused[1])
                return None
            return ops.postnorm_add_norm(resid, out, fused[0], fused[1], nxt[0], nxt[1],
                                         self.ctx.dtype)
        # another kind of norm: its own forward, the add through the next norm (or, with
        # none to follow, through the same norm once more, whose output is dropped)
        normed = post.forward(out)
        if then is not None:
            return then.add_forward(resid, normed)
        post.add_forward(resid, normed)
        return None

    def forward(self, resid, delta, batch, cache, write_cache, next_hint=None):
        if delta is not None:
            # a block in front that hands on a delta (this one gives no entry hint, so it is
            # a plain tensor): added through the mixer's norm, whose output is not used
            self.mixer_norm.add_forward(resid, delta)
        if self.mixer_filter is not None:
            h = self.mixer_filter.forward_from_stream(resid, self.mixer_norm, batch, cache)
        else:
            h = self.mixer_norm.forward(resid)
        out = self.mixer.forward(h, batch, cache, write_cache)
        if self.feed_forward is None:
            self._post_add(resid, out, self.mixer_post_norm)
            return resid, None
        h = self._post_add(resid, out, self.mixer_post_norm, then=self.ffn_norm)
        out = self.feed_forward.forward(h, batch)
        self._post_add(resid, out, self.ffn_post_norm)
        return resid, None


@register(BLOCKS, "parallel_residual")
class ParallelResidualBlock(Block):
    """One norm whose output both sub-layers read: with h = norm(x),
    x <- x + (mixer(h) + ffn(h)).  The feed-forward may be left out.  The stream leaves the
    block summed up (no delta is handed on); where a block of this kind follows, the sum and
    that block's norm (and a row that enters in front of it) are one kernel, and the normed
    rows travel in delta's place."""

    ROLES = {"mixer_norm": (NORMS, True), "mixer": (MIXERS, True),
             "feed_forward": (FEED_FORWARDS, False)}

    def entry_hint(self):
        fused = fused_rmsnorm_of(self.mixer_norm)
        if fused is None or not hasattr(self.ctx.ops, "stream_add_norm"):
            return None
        return NormAhead(fused[0], fused[1])

    def forward(self, resid, delta, batch, cache, write_cache, next_hint=None):
        if isinstance(delta, NormedRows):
            h = delta.rows
        else:
            h = self.mixer_norm.forward(resid) if delta is None \
                else self.mixer_norm.add_forward(resid, delta)
        mixed = self.mixer.forward(h, batch, cache, write_cache)
        fed = self.feed_forward.forward(h, batch) if self.feed_forward is not None else None
        if isinstance(next_hint, NormAhead):
            rows = self.ctx.ops.stream_add_norm(resid, mixed, fed, next_hint.row,
                                                next_hint.norm_weight, next_hint.eps,
                                                self.ctx.dtype)
            return resid, NormedRows(rows, next_hint.row is not None)
        self.ctx.ops.stream_add(resid, mixed, fed, None)
        return resid, None


@register(FILTERS, "token_shift")
class TokenShift(StreamFilter):
    """h_t <- h_t + (h_(t-1) - h_t) * w, element by element, with h the norm of the stream
    and h_(t-1) the previous token's h before this replacement (zeros in front of a
    sequence's first token).  The last token's h (float32) is kept in the request's state
    slot between steps.

    params: weight (tensor name), dim."""

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        self.name, self.dim = params["weight"], int(params["dim"])
        self.weight = None

    def tensors(self):
        return {self.name: TensorDecl((self.dim,), role="vector", init=(0.0, 1.0))}

    def load(self, get):
        self.weight = get(self.name)

    def cache_need(self):
        return SlotStateNeed((self.dim,), torch.float32, "shift")

    def forward_from_stream(self, resid, norm, batch, cache):
        fused = fused_rmsnorm_of(norm)
        if fused is None:
            raise ValueError("token_shift is built behind an RMS norm")
        if cache is None or "shift" not in cache.states:
            raise RuntimeError("token_shift needs its per-request state")
        return self.ops.norm_token_shift(resid, fused[0], fused[1], self.weight, batch,
                                         cache.states["shift"], self.ctx.dtype)
