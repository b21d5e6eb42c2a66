"""How norm, mixer and feed-forward are arranged in a layer (reference models/qwen3.py:55-74)."""
from __future__ import annotations

from .base import FeedForward, Mixer, Norm, Part, PendingNorm, register_part


def norm_of(norm: Norm, x, residual):
    """Run a norm on x, which may be float32 partial sums [P, T, n] of a split product; a norm
    that does not declare `accepts_partials` gets their sum."""
    if x.dim() == 3 and not getattr(norm, "accepts_partials", False):
        x = x.sum(0)
    return norm.forward(x, residual)


@register_part("block", "pre_norm")
class PreNormBlock(Part):
    """residual += input; x = norm1(residual); a = mixer(x); residual += a; x = norm2(residual);
    return feed_forward(x), residual.

    The layer's output is added to the residual by whoever runs next: the next block's first
    norm or the model's final norm (reference models/qwen3.py:65-74: the add lives inside the
    norm call). The residual stream is float32.
    """

    def __init__(self, norm1: Norm, mixer: Mixer, norm2: Norm, feed_forward: FeedForward):
        super().__init__()
        self.add_child("norm1", norm1)
        self.add_child("mixer", mixer)
        self.add_child("norm2", norm2)
        self.add_child("feed_forward", feed_forward)

    def cache_need(self):
        return self.mixer.cache_need()

    def state_need(self):
        return self.mixer.state_need()

    def forward(self, h, residual, step, cache, state):
        # a part that takes it gets the norm before it as a `PendingNorm` and may run it inside its first product
        if getattr(self.mixer, "takes_pending_norm", False):
            x = PendingNorm(self.norm1, h, residual)
            a = self.mixer.forward(x, step, cache, state)
            residual = x.new_residual()
        else:
            x, residual = norm_of(self.norm1, h, residual)
            a = self.mixer.forward(x, step, cache, state)
        if getattr(self.feed_forward, "takes_pending_norm", False):
            x = PendingNorm(self.norm2, a, residual)
            out = self.feed_forward.forward(x)
            return out, x.new_residual()
        x, residual = norm_of(self.norm2, a, residual)
        return self.feed_forward.forward(x), residual
