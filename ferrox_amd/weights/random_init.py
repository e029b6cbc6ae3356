"""Seeded random weights.

Element i of tensor `name` is a function of (seed, name, i) alone: a 64-bit mix
of the counter gives two uniforms, Box-Muller gives a normal.  The same tensors
come out on the CPU and on the GPU, whole or in pieces, for every dtype (values
are made in float32 and rounded).  Matrices, biases and gates are N(0, std^2),
norm weights are 1.  (The reference's own random model, a xorshift stream in
file order, ferrox-models/src/decoder.rs:373-514, is not reproduced.)
"""
from __future__ import annotations

import hashlib
import math

import torch

_M1 = 0xBF58476D1CE4E5B9 - (1 << 64)
_M2 = 0x94D049BB133111EB - (1 << 64)
_GOLD = 0x9E3779B97F4A7C15 - (1 << 64)


def _lsr(x: torch.Tensor, n: int) -> torch.Tensor:
    return (x >> n) & ((1 << (64 - n)) - 1)


def _mix(x: torch.Tensor) -> torch.Tensor:
    """splitmix64 finaliser on int64 tensors (multiplication wraps)."""
    x = (x ^ _lsr(x, 30)) * _M1
    x = (x ^ _lsr(x, 27)) * _M2
    return x ^ _lsr(x, 31)


def _name_key(seed: int, name: str) -> int:
    d = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    v = int.from_bytes(d[:8], "little")
    return v - (1 << 64) if v >= (1 << 63) else v


def normal_values(seed: int, name: str, start: int, count: int, std: float, device) -> torch.Tensor:
    """float32 values [start, start+count) of the stream of tensor `name`."""
    idx = torch.arange(start, start + count, dtype=torch.int64, device=device)
    base = idx * 2 + _name_key(seed, name)
    a = _mix(base * _GOLD + 1)
    b = _mix((base + 1) * _GOLD + 1)
    u1 = (_lsr(a, 40).to(torch.float32) + 0.5) * (1.0 / (1 << 24))
    u2 = (_lsr(b, 40).to(torch.float32) + 0.5) * (1.0 / (1 << 24))
    return torch.sqrt(-2.0 * torch.log(u1)) * torch.cos((2.0 * math.pi) * u2) * std


def random_tensor(seed: int, name: str, spec, dtype: torch.dtype, device, std: float = 0.02,
                  chunk: int = 1 << 24) -> torch.Tensor:
    count = 1
    for d in spec.shape:
        count *= d
    if spec.integer:
        return torch.zeros(spec.shape, dtype=torch.int32, device=device)
    if spec.init == "ones":
        return torch.ones(spec.shape, dtype=dtype, device=device)
    if spec.init == "zeros":
        return torch.zeros(spec.shape, dtype=dtype, device=device)
    out = torch.empty(count, dtype=dtype, device=device)
    for s in range(0, count, chunk):
        n = min(chunk, count - s)
        out[s:s + n] = normal_values(seed, name, s, n, std, device).to(dtype)
    return out.reshape(spec.shape)


class RandomSource:
    """A weight source that makes every tensor a model asks for."""

    def __init__(self, seed: int, dtype: torch.dtype = torch.bfloat16, device="cpu", std: float = 0.02):
        self.seed, self.dtype, self.device, self.std = int(seed), dtype, torch.device(device), float(std)
        self._specs: dict = {}

    def expect(self, specs: dict) -> None:
        self._specs = dict(specs)

    def names(self):
        return list(self._specs)

    def info(self, name):
        spec = self._specs[name]
        return (torch.int32 if spec.integer else self.dtype), tuple(spec.shape)

    def tensor(self, name):
        return random_tensor(self.seed, name, self._specs[name], self.dtype, self.device, self.std)
