"""Arrangements of parts in a block.  Pre-norm (``crates/mach-model/src/batched.rs:3180-3200,
4031, 4050, 4453``): ``x += mixer(norm(x)); x += feed_forward(norm(x))``."""
from __future__ import annotations

from .base import Block
from .registry import FEED_FORWARDS, MIXERS, NORMS, register_block


@register_block("prenorm")
class PreNormBlock(Block):
    """Reads ``mixer``, ``feed_forward``, ``mixer_norm`` and ``feed_forward_norm`` of its layer's spec."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.mixer = MIXERS.build(spec.mixer, rt)
        self.feed_forward = FEED_FORWARDS.build(spec.feed_forward, rt)
        self.mixer_norm = NORMS.build(spec.mixer_norm, rt)
        self.feed_forward_norm = NORMS.build(spec.feed_forward_norm, rt)

    def parts(self):
        return [self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward]

    def forward(self, stream, ctx):
        self.mixer.forward(self._input(self.mixer_norm, self.mixer, stream), stream, ctx)
        self.feed_forward.forward(self._input(self.feed_forward_norm, self.feed_forward, stream), stream, ctx)

    @staticmethod
    def _input(norm, reader, stream):
        """The reader's normalised input: a tensor, or for a reader that starts with a product over it
        the norm left pending, so that the product's kernel can apply it."""
        if reader.takes_pending_norm:
            pending = norm.pending(stream)
            if pending is not None:
                return pending
        return norm.forward(stream)
