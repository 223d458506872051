"""Arrangements of a layer's parts around the residual stream.

Pre-norm with two residual additions, as the reference's block
(/root/reference/src/models/block.cpp:23-29): a = x + Mixer(N1(x)); y = a + FF(N2(a)).
The additions are made in float32 inside the following norm's kernel.
"""
from __future__ import annotations

from .base import Block, PendingNorm, register_part


class PreNormBlock(Block):
    norm_slots = ("mixer", "feed_forward")

    def forward(self, h, delta, ctx, cache, state):
        pending = PendingNorm(h, delta, self.norms["mixer"])                  # x = N1(h + delta)
        x = pending if self.mixer.takes_pending_norm else pending.materialize()
        a = self.mixer.forward(x, ctx, cache, state)
        h = pending.h_after
        pending = PendingNorm(h, a, self.norms["feed_forward"])               # x = N2(h + a)
        x = pending if self.feed_forward.takes_pending_norm else pending.materialize()
        m = self.feed_forward.forward(x, ctx)
        return pending.h_after, m                                            # m is added by whoever comes next


register_part("block", "pre_norm", PreNormBlock)
