"""Arrangements of mixer, feed-forward and norms around the 32-bit residual stream."""

from __future__ import annotations

from .base import Block, register_block


@register_block("prenorm")
class PreNormBlock(Block):
    """x += mixer(norm1(x)); x += feed_forward(norm2(x)) (src/model.cpp:281-305)."""

    roles = {"mixer_norm": "norm", "ffn_norm": "norm", "mixer": "mixer", "feed_forward": "feed_forward"}
    graph_safe = True
    launches_through_ops = True

    def forward(self, ctx, call, x) -> None:
        if not self.mixer.forward_with_norm(ctx, call, x, self.mixer_norm, x):
            h = self.mixer_norm.forward(ctx, x)
            self.mixer.forward(ctx, call, h, x)
        if not self.feed_forward.forward_with_norm(ctx, x, self.ffn_norm, x):
            h = self.ffn_norm.forward(ctx, x)
            self.feed_forward.forward(ctx, h, x)
