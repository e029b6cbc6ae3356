"""Arrangements of a mixer, a feed-forward and norms in one layer."""
from __future__ import annotations

from .base import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, Block


@BLOCKS.register("prenorm")
class PreNormBlock(Block):
    """h += mixer(norm1(h)); h += ffn(norm2(h))   (ferrox-models/src/decoder.rs:1-5, 2155-2173)."""
    slots = {"norm1": NORMS, "mixer": MIXERS, "norm2": NORMS, "ffn": FEED_FORWARDS}

    def __init__(self, parts: dict, prefixes: dict):
        self.norm1, self.mixer, self.norm2, self.ffn = parts["norm1"], parts["mixer"], parts["norm2"], parts["ffn"]
        self._prefixes = prefixes

    def children(self):
        return [(self._prefixes[s], getattr(self, s)) for s in ("norm1", "mixer", "norm2", "ffn")]

    def forward(self, h, ctx, cache) -> None:
        # a part may offer `forward_from_residual(norm, ...)`: it then applies the norm itself, fused
        # into its first kernel, and says False when it cannot for this step
        fused = getattr(self.mixer, "forward_from_residual", None)
        if fused is None or not fused(self.norm1, ctx, cache, h):
            self.mixer.forward(self.norm1.forward(h, ctx), ctx, cache, h)
        fused = getattr(self.ffn, "forward_from_residual", None)
        if fused is None or not fused(self.norm2, ctx, h):
            self.ffn.forward(self.norm2.forward(h, ctx), ctx, h)
