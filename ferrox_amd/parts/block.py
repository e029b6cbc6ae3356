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
        x = self.norm1.forward(h, ctx)
        self.mixer.forward(x, ctx, cache, h)
        x = self.norm2.forward(h, ctx)
        self.ffn.forward(x, ctx, h)
