"""Arrangements of a layer's parts around the 32-bit residual stream.

"prenorm": ``x += mixer(norm(x)); x += feed_forward(norm(x))`` — norm, projections,
rotation, cache write, attention, output, add, norm, feed-forward, add, every layer
alike (src/model.c:6168-6473).

"prenorm_filtered": the same, but what each sublayer reads goes through a sequence filter first:
``x += mixer(filter_m(norm(x))); x += feed_forward(filter_f(norm(x)))``.  A layer of it may come
without a feed-forward.
"""
from __future__ import annotations

from .base import Block, register_block


def _takes_unscaled(part) -> bool:
    return bool(getattr(part, "takes_unscaled_rows", False))


class PreNormBlock(Block):
    chained = True
    norm_names = ("mixer_norm", "feed_forward_norm")

    @property
    def mixer_norm(self):
        return self.norms["mixer_norm"]

    @property
    def feed_forward_norm(self):
        return self.norms["feed_forward_norm"]

    def entry_norm(self):
        return self.mixer_norm, _takes_unscaled(self.mixer)

    def forward(self, ctx, cache, x, h=None, after=None):
        """``h``: the result of ``mixer_norm`` if the block before made it.  ``after``: the next
        block's ``entry_norm()``, whose result is then returned.  The parts' optional
        ``forward_add_norm`` is used where they have it."""
        if h is None:
            h = self.mixer_norm.forward(ctx, x)
        add_norm = getattr(self.mixer, "forward_add_norm", None)
        if add_norm is not None:
            h = add_norm(ctx, cache, h, x, self.feed_forward_norm, defer=_takes_unscaled(self.feed_forward))
        else:
            self.mixer.forward_add(ctx, cache, h, x)
            h = self.feed_forward_norm.forward(ctx, x)
        add_norm = getattr(self.feed_forward, "forward_add_norm", None)
        if after is None or add_norm is None:
            self.feed_forward.forward_add(ctx, h, x)
            return None
        next_norm, defer = after
        return add_norm(ctx, h, x, next_norm, defer=defer)


class FilteredPreNormBlock(Block):
    norm_names = ("mixer_norm", "feed_forward_norm")
    filter_names = ("mixer_filter", "feed_forward_filter")
    needs_feed_forward = None       # with or without; the second norm and filter then do nothing

    def _read(self, ctx, cache, x, norm: str, flt: str):
        """What a sublayer reads: the norm of ``x`` through the filter, in one kernel if the filter has one."""
        f, state = self.filters[flt], cache.states.get(flt)
        fused = getattr(f, "forward_normed", None)
        h = fused(ctx, state, x, self.norms[norm]) if fused is not None else None
        if h is None:
            h = f.forward(ctx, state, self.norms[norm].forward(ctx, x))
        return h

    def forward(self, ctx, cache, x):
        self.mixer.forward_add(ctx, cache, self._read(ctx, cache, x, "mixer_norm", "mixer_filter"), x)
        if self.feed_forward is not None:
            self.feed_forward.forward_add(ctx, self._read(ctx, cache, x, "feed_forward_norm", "feed_forward_filter"), x)

    def state_specs(self):
        out = super().state_specs()
        if self.feed_forward is None:
            out.pop("feed_forward_filter", None)
        return out


register_block("prenorm", PreNormBlock)
register_block("prenorm_filtered", FilteredPreNormBlock)
