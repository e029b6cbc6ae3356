"""Arrangements of a mixer, a feed-forward and norms in one layer."""
from __future__ import annotations

from .. import debug
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

    chains_norms = True     # forward takes `normed` and `then` and returns what the next block may take as `normed`

    @property
    def first_norm(self):
        return self.norm1

    def takes_scale_later(self, act_dtype) -> bool:
        return bool(self.mixer.takes_scale_later(act_dtype))

    def forward(self, h, ctx, cache, normed=None, then=None):
        """`normed`: norm1(h), if the block before has already made it (a tensor, or an ops.ScaleLater if this
        block's mixer takes one).  `then`: (the norm that the next block applies first, whether its mixer
        takes an ops.ScaleLater); a feed-forward that says `norms_after` may apply that norm to the rows it
        has just finished and leave the result in ctx.carry, which is returned (else None)."""
        # a part may offer `forward_from_residual(norm, ...)`: it then applies the norm itself, fused
        # into its first kernel, and says False when it cannot for this step
        if normed is not None:
            self.mixer.forward(normed, ctx, cache, h)
        elif not self.mixer.forward_from_residual(self.norm1, ctx, cache, h):
            debug.region("norm")
            self.mixer.forward(self.norm1.forward(h, ctx), ctx, cache, h)
        ctx.carry = None
        more = {"then_norm": then} if then is not None and self.ffn.norms_after else {}
        if not self.ffn.forward_from_residual(self.norm2, ctx, h, **more):
            debug.region("norm")
            self.ffn.forward(self.norm2.forward(h, ctx), ctx, h, **more)
        out, ctx.carry = ctx.carry, None
        return out
