"""How a norm, a mixer, a second norm and a feed-forward are arranged in a layer.

PreNormBlock:  x <- x + mixer(norm1(x));  x <- x + ff(norm2(x))  (no post-norms),
crates/synaptix-models/llm/common/src/model.rs:1179-1199.  The residual stream x is float; each
sum x + delta is fused into the norm that follows it, so a block returns its last delta
unsummed and takes the previous block's.
"""
from __future__ import annotations

from .base import Part
from .linear import as_rows, as_delta


class Block(Part):
    """Interface: forward(resid, pending, ctx, cache, owner) -> pending.
    resid [N, hidden] float is updated in place; pending is a delta not yet added (or None)."""

    mixer = None
    # True: `pending` may arrive as a parts.linear.DeferredProduct (a product that the block's first norm can take
    # in); False (the default): the model runs such a product before it calls the block
    takes_deferred_product = False

    def forward(self, resid, pending, ctx, cache, owner=True):
        raise NotImplementedError


def _norm_input(norm, delta):
    return delta if getattr(norm, "takes_deferred_product", False) else as_delta(delta)


class PreNormBlock(Block):
    takes_deferred_product = True

    def __init__(self, norm1, mixer, norm2, feed_forward):
        self.norm1, self.mixer, self.norm2, self.feed_forward = norm1, mixer, norm2, feed_forward

    def _parts(self):
        return (self.norm1, self.mixer, self.norm2, self.feed_forward)

    @property
    def capturable(self):
        return all(getattr(p, "capturable", False) for p in self._parts())

    def tensor_specs(self):
        specs = {}
        for p in self._parts():
            specs.update(p.tensor_specs())
        return specs

    def load(self, get):
        for p in self._parts():
            p.load(get)

    def check(self, dtype):
        for p in self._parts():
            p.check(dtype)

    def forward(self, resid, pending, ctx, cache, owner=True):
        # a norm may hand on rows whose last step a product finishes, and take a product that has not been run
        # (parts.linear.ScaledRows, DeferredProduct); parts that do not say they take them get plain tensors
        h = self.norm1.add_apply(resid, _norm_input(self.norm1, pending), ctx.act_dtype)
        a = self.mixer.forward(h if self.mixer.takes_scaled_rows else as_rows(h), ctx, cache, owner)
        h2 = self.norm2.add_apply(resid, _norm_input(self.norm2, a), ctx.act_dtype)
        return self.feed_forward.forward(h2 if self.feed_forward.takes_scaled_rows else as_rows(h2), ctx)
