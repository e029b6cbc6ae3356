"""Sampling parameters, the per-request generator, and the batched call into the
sampling kernel.

Options and their meaning are the reference's `SamplingParams`
(ferrox-models/src/sampling.rs:17-52): temperature <= 0 is greedy; top_k 0 and
top_p 1.0 are off; repetition_penalty 1.0 is off; presence and frequency
penalties 0 are off.  Each request owns a xorshift64 generator seeded from its
seed (sampling.rs:66-84), advanced once per sampled token, so a request draws
the same numbers whatever it is batched with
(ferrox-server/src/batch_scheduler.rs:304, 404-451).
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .. import ops

_MASK = (1 << 64) - 1


@dataclass
class SamplingParams:
    temperature: float = 0.0
    top_k: int = 0
    top_p: float = 1.0
    repetition_penalty: float = 1.0
    presence_penalty: float = 0.0
    frequency_penalty: float = 0.0
    seed: int = 0

    @property
    def greedy(self) -> bool:
        return self.temperature <= 0.0

    @property
    def uses_history(self) -> bool:
        return self.repetition_penalty != 1.0 or self.presence_penalty != 0.0 or self.frequency_penalty != 0.0


class XorShift64:
    """Shifts 13, 7, 17; a zero seed is replaced (sampling.rs:66-78)."""

    def __init__(self, seed: int):
        seed &= _MASK
        self.state = 0x9E3779B97F4A7C15 if seed == 0 else seed

    def next_u64(self) -> int:
        s = self.state
        s ^= (s << 13) & _MASK
        s ^= s >> 7
        s ^= (s << 17) & _MASK
        self.state = s
        return s

    def next_f32(self) -> float:
        """Uniform in [0, 1) with 24 bits (sampling.rs:81-84)."""
        return (self.next_u64() >> 40) / float(1 << 24)


def _upload(dev, floats: dict, ints: dict) -> dict:
    """All per-row parameters of one sampling call in one pinned buffer and one copy that the host does not wait
    for: name -> float32 or int32 tensor on `dev`."""
    n = sum(len(v) for v in floats.values()) + sum(len(v) for v in ints.values())
    host = torch.empty(n, dtype=torch.float32, pin_memory=True)
    as_f, as_i = host.numpy(), host.view(torch.int32).numpy()
    spans, o = {}, 0
    for group, view, integer in ((floats, as_f, False), (ints, as_i, True)):
        for name, vals in group.items():
            view[o:o + len(vals)] = vals
            spans[name] = (o, o + len(vals), integer)
            o += len(vals)
    there = host.to(dev, non_blocking=True)
    there_i = there.view(torch.int32)
    return {name: (there_i if integer else there)[a:b] for name, (a, b, integer) in spans.items()}


def launch_sample_rows(logits: torch.Tensor, params: list, rngs: list, histories: list) -> torch.Tensor:
    """One token id per row of `logits` [R, V] (float32, on the GPU), as an int32 tensor on the GPU; the host
    waits for nothing.  `params[r]`, `rngs[r]`, `histories[r]` (the tokens generated so far) belong to row r.
    A generator is advanced only for rows that draw."""
    if all(p.greedy and not p.uses_history for p in params):
        return ops.sample(logits)
    draws = [0.0 if p.greedy else rng.next_f32() for p, rng in zip(params, rngs)]
    floats, ints = dict(temperature=[p.temperature for p in params], draw=draws), {}
    if any(p.top_k > 0 for p in params):
        ints["top_k"] = [p.top_k for p in params]
    if any(p.top_p < 1.0 for p in params):
        floats["top_p"] = [p.top_p for p in params]
    if any(p.uses_history for p in params):
        flat, starts = [], [0]
        for p, h in zip(params, histories):
            if p.uses_history:
                flat.extend(h)
            starts.append(len(flat))
        ints["hist"], ints["hist_start"] = flat or [0], starts
        floats["rep_penalty"] = [p.repetition_penalty for p in params]
        floats["presence"] = [p.presence_penalty for p in params]
        floats["frequency"] = [p.frequency_penalty for p in params]
    return ops.sample(logits, **_upload(logits.device, floats, ints))


def sample_rows(logits: torch.Tensor, params: list, rngs: list, histories: list, launched=None) -> list:
    """`launch_sample_rows`, read back: a list of token ids.  `launched()` is called after the kernel is
    launched and before the host waits for the ids (for measurement)."""
    out = launch_sample_rows(logits, params, rngs, histories)
    if launched is not None:
        launched()
    return out.tolist()
