"""Pre-norm block with the residual adds deferred into the norms.

stream += pending; y = norm1(stream); a = mixer(y); stream += a; y = norm2(stream);
pending' = feed_forward(y).  The block returns its feed-forward output still to
be added: the next block's first norm (or the final norm) adds it
(inference_engine/model.py:169-171,179,184).
"""
from __future__ import annotations

from ..kernels.api import Sink
from .base import Block, register_block


@register_block("pre_norm")
class PreNormBlock(Block):
    def __init__(self, norm_mixer, mixer, norm_feed_forward, feed_forward):
        self.norm_mixer = norm_mixer
        self.mixer = mixer
        self.norm_feed_forward = norm_feed_forward
        self.feed_forward = feed_forward

    def children(self):
        return [self.norm_mixer, self.mixer, self.norm_feed_forward, self.feed_forward]

    @property
    def first_norm(self):
        return self.norm_mixer

    def forward(self, h, residual, step, cache, next_norm=None):
        """``next_norm``: the norm that reads the stream after this block (the next block's first norm or
        the model's final norm), if the model knows it."""
        y = self.norm_mixer.lazy(h, residual)
        if not self.mixer.lazy_input:
            y = y.materialize()
        a = self.mixer.forward(y, step, cache, add_to=_sink(residual, self.norm_feed_forward))
        y = self.norm_feed_forward.lazy(a, residual)
        if not self.feed_forward.lazy_input:
            y = y.materialize()
        return self.feed_forward.forward(y, step, add_to=_sink(residual, next_norm)), residual


def _sink(residual, norm):
    weight, eps = getattr(norm, "weight", None), getattr(norm, "eps", None)
    if weight is None or eps is None:
        return Sink(residual)
    return Sink(residual, weight, eps)
