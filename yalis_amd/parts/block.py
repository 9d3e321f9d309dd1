"""Block arrangements: how norms, mixer and feed-forward sit around the residual.

"prenorm" is the reference's sequential pre-norm block
(yalis/external/model.py:414-439 with parallel_residual=False and identity
post-norms): x = x + mixer(norm_1(x)); x = x + feed_forward(norm_2(x)).

The residual stream is float32.  A block receives the residual and the previous
block's not-yet-added contribution ``delta``; each norm kernel adds the pending
contribution and normalises in one pass, so no separate addition runs.  The block
returns its own last contribution, to be added by whoever comes next.
"""
from __future__ import annotations

from .base import Block, register_block


@register_block("prenorm")
class PreNormBlock(Block):
    roles = {
        "mixer_norm": ("norm", True),
        "mixer": ("mixer", True),
        "feed_forward_norm": ("norm", True),
        "feed_forward": ("feed_forward", True),
    }

    def __init__(self, mixer_norm, mixer, feed_forward_norm, feed_forward):
        self.mixer_norm = mixer_norm
        self.mixer = mixer
        self.feed_forward_norm = feed_forward_norm
        self.feed_forward = feed_forward

    @property
    def takes_embedded_rows(self):
        return bool(getattr(self.mixer_norm, "takes_embedded_rows", False))

    def forward(self, residual, delta, ctx, site):
        h = self.mixer_norm.add_norm(residual, delta)
        a = self.mixer.forward(h, ctx, site)
        h = self.feed_forward_norm.add_norm(residual, a)
        return self.feed_forward.forward(h, ctx)
