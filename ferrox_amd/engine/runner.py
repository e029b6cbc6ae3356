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

import gc

from dataclasses import dataclass, field

import torch

from .. import debug, ops
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
        total = mgr.step_words(n_seqs, n_seqs, n_seqs, self.max_blocks)
        dev = runner.device
        # behind the step's own words: room for one (place, row) pair per token that is fed from the device
        self.meta = torch.zeros(total + 2 * n_seqs, dtype=torch.int32, device=dev)
        self.host = torch.zeros(total + 2 * n_seqs, dtype=torch.int32, pin_memory=True)
        self._host_ptr, self._host_words = self.host.data_ptr(), total
        self._host_np = self.host.numpy()
        self.copied = torch.cuda.Event()
        self.copied.record()
        self.graph = None
        self.logits = None
        self.trace_calls = None        # where an active routing trace's copies went while this step was recorded

    def _context(self) -> StepContext:
        n, mb, m = self.n, self.max_blocks, self.meta
        tables, o = {}, 5 * n
        for key in self.keys:
            tables[key] = m[o:o + n * mb].view(n, mb)
            o += n * mb
        ctx = StepContext(n_tokens=n, n_seqs=n, act_dtype=self.runner.act_dtype, device=self.runner.device,
                          token_ids=m[0:n], positions=m[n:2 * n], token_seq=m[2 * n:3 * n],
                          q_starts=list(range(n + 1)), kv_lens=[self.kv_bound] * n, slot_ids=m[3 * n:4 * n],
                          slots=None, block_tables=tables, block_size=self.runner.block_size,
                          logit_rows=m[4 * n:5 * n], recorded=True, kv_bound=self.kv_bound)
        return ctx

    def run(self, entries, feed=None) -> torch.Tensor:
        """The logits of the entries' tokens (one each).  Fewer entries than the step was recorded for are
        filled up with stand-in rows, which write to a page and a slot that no request owns.  `feed` as in
        `ModelRunner.step`."""
        self.copied.synchronize()                  # the last upload has left the staging buffer
        for e in entries:
            if e.want[0] != 0:
                raise ValueError(f"request {e.req!r}: wanted place {e.want[0]} is outside its one token")
        storage = self.runner.storage
        self.runner.manager.pack_decode([e.req for e in entries], [e.tokens[0] for e in entries], self.runner.vocab_size,
                                        self._host_ptr, self._host_words, self.max_blocks, pad_to=self.n,
                                        pad_pages=storage.pad_pages, pad_slot=storage.pad_slot)
        if self.runner.before_launch is not None:
            self.runner.before_launch()
        words = self._host_words
        if feed:
            ids, pairs = feed
            flat = check_feed(ids, pairs, len(entries))
            self._host_np[words:words + len(flat)] = flat
            self.meta[:words + len(flat)].copy_(self.host[:words + len(flat)], non_blocking=True)
            ops.feed_tokens(self.meta[:self.n], ids, self.meta[words:words + len(flat)].view(-1, 2),
                            len(entries), ids.numel())
        else:
            self.meta[:words].copy_(self.host[:words], non_blocking=True)
        self.copied.record()
        model, caches = self.runner.model, self.runner.storage.caches
        if self.graph is None:
            model.forward(self._context(), caches)              # once eagerly: loads the kernels
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            # no garbage collection while the stream is recording: a tensor of an earlier step that is freed
            # then makes the allocator query events, which a recording stream does not allow
            collecting = gc.isenabled()
            gc.disable()
            if debug.routing_trace is not None:
                debug.routing_trace.begin_step()     # the recorded launches write where the eager ones just wrote
            # (capture_begin / capture_end on a stream of its own rather than `with torch.cuda.graph(...)`: that
            # context manager also gives the allocator's cached memory back to the driver first, which with tens of
            # GB in the cache costs a recording several hundred milliseconds)
            main, side = torch.cuda.current_stream(), self.runner.capture_stream
            side.wait_stream(main)
            try:
                with torch.cuda.stream(side):
                    graph.capture_begin()
                    try:
                        self.logits = model.forward(self._context(), caches)
                    finally:
                        graph.capture_end()
            finally:
                if collecting:
                    gc.enable()
            main.wait_stream(side)
            self.graph = graph
            if debug.routing_trace is not None:
                self.trace_calls = debug.routing_trace.calls()
        self.graph.replay()
        if debug.routing_trace is not None:
            debug.routing_trace.replayed(self.trace_calls)
        return self.logits[:len(entries)]


def check_feed(ids: torch.Tensor, pairs: list, n_tokens: int) -> list:
    """`pairs` flattened, after a check that every place lies among the step's tokens and every row among `ids`."""
    flat = []
    for place, row in pairs:
        if not (0 <= place < n_tokens and 0 <= row < ids.numel()):
            raise ValueError(f"token {place} of {n_tokens} cannot be fed from row {row} of {ids.numel()} sampled ids")
        flat += (place, row)
    return flat


class ModelRunner:
    def __init__(self, model, *, block_size: int = 64, num_pages: int = 64, max_seqs: int = 8,
                 use_graphs: bool = True, graph_kv_step: int = 512):
        if model.device is None:
            raise RuntimeError("load the model's weights before making a runner")
        if model.device.type != "cuda":
            raise RuntimeError("the engine runs on the GPU only; there is no CPU path")
        ensure_built(list(model.kernel_libraries()) + ["host_runtime"])
        self.model = model
        self.act_dtype, self.device = model.act_dtype, model.device
        self.block_size = block_size
        self.manager = CacheManager(model.cache_groups(), num_pages, block_size, max_seqs)
        self.storage = CacheStorage(model, self.manager, self.act_dtype, self.device)
        self.vocab_size = model.spec.vocab_size
        # decode steps are replayed from HIP graphs if every mixer can be recorded
        self.use_graphs = use_graphs and all(b.mixer.graph_safe for b in model.blocks)
        self.graph_kv_step = graph_kv_step
        self.capture_stream = torch.cuda.Stream(device=self.device) if use_graphs else None     # default priority
        self._graphs: dict = {}
        self._host = None                      # pinned staging buffer of the step's int32 data
        self.before_launch = None              # measurement: called right before a step's first device operation
        self._uploaded = torch.cuda.Event()

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
    def _staging(self, words: int) -> torch.Tensor:
        """A pinned host buffer of at least `words` int32 that no upload is still reading."""
        if self._host is None or self._host.numel() < words:
            self._host = torch.zeros(max(4096, 2 * words), dtype=torch.int32, pin_memory=True)
        else:
            self._uploaded.synchronize()
        return self._host

    def step(self, entries: list, feed=None) -> torch.Tensor | None:
        """Logits [number of wanted places, vocab] in the order of the entries and of each
        entry's `want`, or None if nothing is wanted.  Every entry's request must hold pages
        for its tokens already (`reserve`).

        `feed = (ids, [(place, row), ...])` names tokens of this step that the host does not know yet: token
        number `place` (counted through all entries) is `ids[row]`, an int32 tensor on the device that an
        earlier step's sampling wrote; the entry holds any valid id in its stead.  So a step can be launched
        while the one before it still runs."""
        mgr = self.manager
        n_seqs = len(entries)
        reqs = [e.req for e in entries]
        token_lists, wants = [e.tokens for e in entries], [e.want for e in entries]
        T, R = sum(len(t) for t in token_lists), sum(len(w) for w in wants)
        if debug.routing_trace is not None:
            debug.routing_trace.begin_step()
        if self.use_graphs and n_seqs and all(len(t) == 1 for t in token_lists) and all(len(w) == 1 for w in wants):
            # every sequence brings one token and wants its logits: a recorded decode step
            longest = max(mgr.length(r) for r in reqs)
            bound = -(-longest // self.graph_kv_step) * self.graph_kv_step
            # more than eight sequences are recorded in steps of eight and filled up with stand-in rows: a batch
            # that shrinks by one request at a time then records a step once in eight times, not every time
            n_rec = n_seqs if n_seqs <= 8 else -(-n_seqs // 8) * 8
            key = (n_rec, bound, debug.graph_token())
            if key in self._graphs:
                self._graphs[key] = self._graphs.pop(key)          # kept in the order of last use
            else:
                if len(self._graphs) >= 32:
                    # the step that goes is the one unused for longest; the device may still be running it (steps
                    # are launched ahead of their results), and its memory goes with it
                    torch.cuda.current_stream(self.device).synchronize()
                    self._graphs.pop(next(iter(self._graphs)))
                self._graphs[key] = DecodeGraph(self, n_rec, bound)
            try:
                logits = self._graphs[key].run(entries, feed)
            except RuntimeError as err:
                # recording is an optimisation of how kernels are launched, not another code path:
                # if the runtime refuses it, the same kernels are launched one by one from here on
                import warnings
                warnings.warn(f"recording decode steps as HIP graphs failed ({err}); launching kernels directly")
                self.use_graphs = False
                self._graphs.clear()
                logits = None
            if logits is not None:
                for r in reqs:
                    mgr.trim(r)
                return logits
        longest = max((mgr.length(r) for r in reqs if r in mgr), default=0)
        max_blocks = max(1, mgr.blocks_for(longest))
        flat = check_feed(feed[0], feed[1], T) if feed else []
        host = self._staging(mgr.step_words(T, n_seqs, R, max_blocks) + len(flat))
        packed = mgr.pack_step(reqs, token_lists, wants, self.vocab_size, host.data_ptr(), host.numel())
        words = packed.total + len(flat)
        if flat:
            host[packed.total:words] = torch.tensor(flat, dtype=torch.int32)
        dev = torch.empty(words, dtype=torch.int32, device=self.device)
        if self.before_launch is not None:
            self.before_launch()
        dev.copy_(host[:words], non_blocking=True)
        self._uploaded.record()
        if flat:
            ops.feed_tokens(dev[:T], feed[0], dev[packed.total:words].view(-1, 2), T, feed[0].numel())
        o = 0

        def take(n):
            nonlocal o
            v = dev[o:o + n]
            o += n
            return v

        mb = packed.max_blocks
        d_tokens, d_pos, d_seq, d_slots, d_rows = take(T), take(T), take(T), take(n_seqs), take(R)
        tables = {key: take(n_seqs * mb).view(n_seqs, mb) for key in mgr.groups}
        q_starts = [0]
        for t in token_lists:
            q_starts.append(q_starts[-1] + len(t))
        ctx = StepContext(n_tokens=T, n_seqs=n_seqs, act_dtype=self.act_dtype, device=self.device,
                          token_ids=d_tokens, positions=d_pos, token_seq=d_seq, q_starts=q_starts,
                          kv_lens=packed.lens, slot_ids=d_slots, slots=host[3 * T:3 * T + n_seqs].tolist(),
                          block_tables=tables, block_size=self.block_size, logit_rows=d_rows if R else None)
        logits = self.model.forward(ctx, self.storage.caches)
        for r in reqs:
            mgr.trim(r)
        return logits
