"""Arrangements of a layer's parts around the residual stream.

Pre-norm with two residual additions, as the reference's block
(/root/reference/src/models/block.cpp:23-29): a = x + Mixer(N1(x)); y = a + FF(N2(a)).
The additions are made in float32 inside the following norm's kernel.
"""
from __future__ import annotations

from .base import Block, register_part


class PreNormBlock(Block):
    def forward(self, h, delta, ctx, cache, state):
        x = self.mixer_norm.forward(h, delta)          # h += delta; x = N1(h)
        a = self.mixer.forward(x, ctx, cache, state)
        x = self.feed_forward_norm.forward(h, a)       # h += a;     x = N2(h)
        return self.feed_forward.forward(x, ctx)       # added by whoever comes next


register_part("block", "pre_norm", PreNormBlock)
