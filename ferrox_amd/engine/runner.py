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


class DecodeGraph:
    """One decode step (every sequence brings one token) recorded as a HIP graph.

    What changes from step to step — tokens, positions, slots, block tables — lives in one
    int32 device buffer at a fixed address that is refreshed before each replay; everything a
    kernel launch depends on beside that (number of sequences, width of the block tables, the
    bound on the sequence lengths that sets the number of attention splits) is fixed per graph.
    """

    def __init__(self, runner, n_seqs: int, kv_bound: int):
        self.runner, self.n, self.kv_bound = runner, n_seqs, kv_bound
        mgr = runner.manager
        self.max_blocks = max(1, mgr.blocks_for(kv_bound))
        self.keys = list(mgr.groups)
        total = 3 * n_seqs + len(self.keys) * n_seqs * self.max_blocks
        dev = runner.device
        self.meta = torch.zeros(total, dtype=torch.int32, device=dev)
        self.host = torch.zeros(total, dtype=torch.int32, pin_memory=True)
        self.copied = torch.cuda.Event()
        self.copied.record()
        self.arange = torch.arange(n_seqs, dtype=torch.int32, device=dev)
        self.graph = None
        self.logits = None

    def _context(self) -> StepContext:
        n, mb = self.n, self.max_blocks
        tables, o = {}, 3 * n
        for key in self.keys:
            tables[key] = self.meta[o:o + n * mb].view(n, mb)
            o += n * mb
        ctx = StepContext(n_tokens=n, n_seqs=n, act_dtype=self.runner.act_dtype, device=self.runner.device,
                          token_ids=self.meta[0:n], positions=self.meta[n:2 * n], token_seq=self.arange,
                          q_starts=list(range(n + 1)), kv_lens=[self.kv_bound] * n, slot_ids=self.meta[2 * n:3 * n],
                          slots=None, block_tables=tables, block_size=self.runner.block_size, logit_rows=self.arange)
        ctx._memo["attention_items"] = {"n_decode": n, "n_tiles": 0, "max_kv": self.kv_bound,
                                        "dec_seq": self.arange, "dec_tok": self.arange}
        return ctx

    def run(self, tokens, positions, slots, table_rows) -> torch.Tensor:
        n, mb = self.n, self.max_blocks
        self.copied.synchronize()                  # the last upload has left the staging buffer
        h = self.host
        h[0:n] = torch.tensor(tokens, dtype=torch.int32)
        h[n:2 * n] = torch.tensor(positions, dtype=torch.int32)
        h[2 * n:3 * n] = torch.tensor(slots, dtype=torch.int32)
        o = 3 * n
        for rows in table_rows:                    # one list of rows per group, in the order of self.keys
            flat = []
            for r in rows:
                flat.extend(max(p, 0) for p in r[:mb])
                flat.extend([0] * (mb - min(len(r), mb)))
            h[o:o + n * mb] = torch.tensor(flat, dtype=torch.int32)
            o += n * mb
        self.meta.copy_(h, non_blocking=True)
        self.copied.record()
        model, caches = self.runner.model, self.runner.storage.caches
        if self.graph is None:
            model.forward(self._context(), caches)              # once eagerly: loads the kernels
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                self.logits = model.forward(self._context(), caches)
            self.graph = graph
        self.graph.replay()
        return self.logits


class ModelRunner:
    def __init__(self, model, *, block_size: int = 64, num_pages: int = 64, max_seqs: int = 8,
                 use_graphs: bool = True, graph_kv_step: int = 512):
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
        # decode steps are replayed from HIP graphs if every mixer can be recorded
        self.use_graphs = use_graphs and all(getattr(b.mixer, "graph_safe", False) for b in model.blocks)
        self.graph_kv_step = graph_kv_step
        self._graphs: dict = {}

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
        if self.use_graphs and T == n_seqs and len(rows) == n_seqs:
            # every sequence brings one token and wants its logits: a recorded decode step
            bound = -(-max(kv_lens) // self.graph_kv_step) * self.graph_kv_step
            key = (n_seqs, bound)
            if key not in self._graphs:
                if len(self._graphs) >= 16:
                    self._graphs.pop(next(iter(self._graphs)))
                self._graphs[key] = DecodeGraph(self, n_seqs, bound)
            try:
                logits = self._graphs[key].run(tokens, positions, slots,
                                               [[mgr.table(e.req, k) for e in entries] for k in mgr.groups])
            except RuntimeError as err:
                # recording is an optimisation of how kernels are launched, not another code path:
                # if the runtime refuses it, the same kernels are launched one by one from here on
                import warnings
                warnings.warn(f"recording decode steps as HIP graphs failed ({err}); launching kernels directly")
                self.use_graphs = False
                self._graphs.clear()
                logits = None
            if logits is not None:
                for e in entries:
                    mgr.trim(e.req)
                return logits
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
