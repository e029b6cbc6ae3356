"""Rotary position encodings.  The attention kernels rotate q and k themselves
while they write the cache, so these parts only carry the constants.

'rope_neox' pairs (i, i + rot/2) — the layout of ferrox-core/src/attention.rs:20-32,
which the reference's registry gives this architecture
(ferrox-models/src/capability.rs:252-258); 'rope_interleaved' pairs (2i, 2i+1)
(attention.rs `apply_rope_interleaved`).  angle = pos * theta^(-2i/rot).
"""
from __future__ import annotations

from .base import POSITION_ENCODINGS, PositionEncoding, Rotary


class _Rotary(PositionEncoding):
    interleaved = False

    def __init__(self, head_dim: int, theta: float, rotary_dim: int | None = None):
        self.head_dim = int(head_dim)
        self.theta = float(theta)
        self.rotary_dim = int(rotary_dim if rotary_dim is not None else head_dim)
        if self.rotary_dim % 2 or not 0 <= self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and at most head_dim {self.head_dim}")
        if not self.theta > 0:
            raise ValueError(f"rope theta must be positive, got {self.theta}")

    def rotary(self):
        return Rotary(self.rotary_dim, self.theta, self.interleaved)


@POSITION_ENCODINGS.register("rope_neox")
class NeoxRope(_Rotary):
    interleaved = False


@POSITION_ENCODINGS.register("rope_interleaved")
class InterleavedRope(_Rotary):
    interleaved = True


@POSITION_ENCODINGS.register("none")
class NoPositions(PositionEncoding):
    def __init__(self, head_dim: int = 0):
        self.head_dim = head_dim

    def rotary(self):
        return Rotary(0, 1.0)
