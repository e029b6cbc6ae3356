"""The step function: one batch of (request, its next tokens) through the model.

A step runs only the tokens it is given, as one batch, against the cache that
earlier steps left, and returns float32 logits at the wanted places.  Portions
of prompts and single decoded tokens may stand side by side, cut anywhere.
(The reference has three separate entry points for a span of one sequence, for
one token and for one token of each of N sequences,
ferrox-models/src/decoder.rs:3014, 1237, 3701; this one call covers them.)
Pages for the step's new positions are taken from the cache manager *before*
the step, by whoever schedules it.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import torch

from ..cache.manager import CacheManager
from ..cache.storage import CacheStorage
from ..csrc.build import ensure_built
from ..parts.base import StepContext


@dataclass
class StepEntry:
    req: object
    tokens: list
    want: list = field(default_factory=list)     # places among `tokens` whose logits are asked for


class ModelRunner:
    def __init__(self, model, *, block_size: int = 64, num_pages: int = 64, max_seqs: int = 8):
        if model.device is None:
            raise RuntimeError("load the model's weights before making a runner")
        if model.device.type != "cuda":
            raise RuntimeError("the engine runs on the GPU only; there is no CPU path")
        ensure_built(model.kernel_libraries())
        self.model = model
        self.act_dtype, self.device = model.act_dtype, model.device
        self.block_size = block_size
        self.manager = CacheManager(model.cache_groups(), num_pages, block_size, max_seqs)
        self.storage = CacheStorage(model, self.manager, self.act_dtype, self.device)
        self.vocab_size = model.spec.vocab_size

    # ---- requests ----------------------------------------------------------
    def admit(self, req) -> bool:
        slot = self.manager.admit(req)
        if slot is None:
            return False
        self.storage.clear_slot(slot)
        return True

    def reserve(self, req, n_new: int) -> bool:
        """Pages for the request's next n_new positions, all or nothing."""
        return self.manager.extend(req, self.manager.length(req) + n_new)

    def release(self, req) -> None:
        self.manager.release(req)

    # ---- the step ----------------------------------------------------------
    def step(self, entries: list) -> torch.Tensor | None:
        """Logits [number of wanted places, vocab] in the order of the entries and of each
        entry's `want`, or None if nothing is wanted.  Every entry's request must hold pages
        for its tokens already (`reserve`)."""
        mgr, bs = self.manager, self.block_size
        tokens, positions, token_seq, q_starts, kv_lens, slots, rows = [], [], [], [0], [], [], []
        for s, e in enumerate(entries):
            n = len(e.tokens)
            if n == 0:
                raise ValueError(f"request {e.req!r} brings no tokens to this step")
            if e.req not in mgr:
                raise ValueError(f"request {e.req!r} was not admitted")
            end = mgr.length(e.req)
            start = end - n
            if start < 0:
                raise ValueError(f"request {e.req!r}: {n} tokens but only {end} positions are reserved")
            for t in e.tokens:
                if not 0 <= int(t) < self.vocab_size:
                    raise ValueError(f"request {e.req!r}: token id {t} is outside the vocabulary "
                                     f"of {self.vocab_size}")     # ferrox-cli/src/run.rs:598-601
            for w in e.want:
                if not 0 <= int(w) < n:
                    raise ValueError(f"request {e.req!r}: wanted place {w} is outside its {n} tokens")
                rows.append(len(tokens) + int(w))
            tokens.extend(int(t) for t in e.tokens)
            positions.extend(range(start, end))
            token_seq.extend([s] * n)
            q_starts.append(len(tokens))
            kv_lens.append(end)
            slots.append(mgr.slot(e.req))
        if len({e.req for e in entries}) != len(entries):
            raise ValueError("a request appears twice in one step")
        n_seqs, T = len(entries), len(tokens)
        max_blocks = max(1, max(mgr.blocks_for(L) for L in kv_lens))
        tables = {}
        flat = tokens + positions + token_seq + slots + rows
        for key in mgr.groups:
            for e in entries:
                t = mgr.table(e.req, key)
                flat.extend(max(p, 0) for p in t[:max_blocks])
                flat.extend([0] * (max_blocks - min(len(t), max_blocks)))
        dev = torch.tensor(flat, dtype=torch.int32).to(self.device, non_blocking=False)
        o = 0

        def take(n):
            nonlocal o
            v = dev[o:o + n]
            o += n
            return v

        d_tokens, d_pos, d_seq, d_slots, d_rows = take(T), take(T), take(T), take(n_seqs), take(len(rows))
        for key in mgr.groups:
            tables[key] = take(n_seqs * max_blocks).view(n_seqs, max_blocks)
        ctx = StepContext(n_tokens=T, n_seqs=n_seqs, act_dtype=self.act_dtype, device=self.device,
                          token_ids=d_tokens, positions=d_pos, token_seq=d_seq, q_starts=q_starts,
                          kv_lens=kv_lens, slot_ids=d_slots, slots=slots, block_tables=tables,
                          block_size=bs, logit_rows=d_rows if rows else None)
        logits = self.model.forward(ctx, self.storage.caches)
        for e in entries:
            mgr.trim(e.req)
        return logits
