"""Arrangements of parts in a block.  Pre-norm (``crates/mach-model/src/batched.rs:3180-3200,
4031, 4050, 4453``): ``x += mixer(norm(x)); x += feed_forward(norm(x))``."""
from __future__ import annotations

from .base import Block
from .registry import register_block


@register_block("prenorm")
class PreNormBlock(Block):
    def forward(self, stream, ctx):
        self.mixer.forward(self.mixer_norm.forward(stream), stream, ctx)
        self.feed_forward.forward(self.feed_forward_norm.forward(stream), stream, ctx)
