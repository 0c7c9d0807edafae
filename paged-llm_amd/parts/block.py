"""Pre-norm residual block: x += mixer(norm1(x)); x += feed_forward(norm2(x))
(pagedllm/model/llama.py:174-185).

The residual stream travels as (x, delta) with delta not yet added, so each norm adds the
previous branch's output in its own kernel; the sum is formed in float and rounded once to the
stream's element type, which is what a plain add in that type gives.
"""

from __future__ import annotations

from .base import Block
from .registry import register_block


class PreNormBlock(Block):
    """params: the four roles' prefixes in tensor names (mixer_norm, mixer, feed_forward_norm, feed_forward)."""
    ROLES = {"mixer_norm": "norm", "mixer": "mixer", "feed_forward_norm": "norm", "feed_forward": "feed_forward"}

    def accepts_partial_delta(self):
        return bool(getattr(self.parts["mixer_norm"], "accepts_partial_sums", False))

    def forward(self, x, delta, ctx, cache, state):
        p = self.parts
        # What a branch returns goes to a norm as its delta.  If that norm can add float partial sums itself, the branch
        # is told so (``ctx.partial_sums_ok``) and may end in a product whose ranges of the inner dimension nobody has
        # added yet; for the feed-forward's output the model says what the next consumer takes.
        after_block = bool(getattr(ctx, "partial_sums_ok", False))
        h = p["mixer_norm"].pending(x, delta)             # summed and normed by whoever consumes it first
        ctx.partial_sums_ok = bool(getattr(p["feed_forward_norm"], "accepts_partial_sums", False))
        a = p["mixer"].forward(h, ctx, cache, state)
        x = h.residual()
        h = p["feed_forward_norm"].pending(x, a)
        ctx.partial_sums_ok = after_block
        m = p["feed_forward"].forward(h, ctx)
        return h.residual(), m


register_block("prenorm", PreNormBlock)
