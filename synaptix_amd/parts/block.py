"""How a norm, a mixer, a second norm and a feed-forward are arranged in a layer.

PreNormBlock:  x <- x + mixer(norm1(x));  x <- x + ff(norm2(x))  (no post-norms),
crates/synaptix-models/llm/common/src/model.rs:1179-1199.  The residual stream x is float; each
sum x + delta is fused into the norm that follows it, so a block returns its last delta
unsummed and takes the previous block's.
"""
from __future__ import annotations

from .base import Part


class Block(Part):
    """Interface: forward(resid, pending, ctx, cache, owner) -> pending.
    resid [N, hidden] float is updated in place; pending is a delta not yet added (or None)."""

    mixer = None

    def forward(self, resid, pending, ctx, cache, owner=True):
        raise NotImplementedError


class PreNormBlock(Block):
    def __init__(self, norm1, mixer, norm2, feed_forward):
        self.norm1, self.mixer, self.norm2, self.feed_forward = norm1, mixer, norm2, feed_forward

    def _parts(self):
        return (self.norm1, self.mixer, self.norm2, self.feed_forward)

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
        h = self.norm1.add_apply(resid, pending, ctx.act_dtype)
        a = self.mixer.forward(h, ctx, cache, owner)
        h2 = self.norm2.add_apply(resid, a, ctx.act_dtype)
        return self.feed_forward.forward(h2, ctx)
