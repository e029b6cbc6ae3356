"""Continuous batching: which requests run in the next step, and with how many tokens.

Every step is one mixed batch under a token budget: each running request that
is decoding brings its one token; what is left of the budget goes to portions of
prompts, oldest request first, each at most `prefill_chunk` long; then waiting
requests are admitted while a state slot, budget and pages for their first
portion are there.  (The reference prefills a whole prompt token by token at
admission and batches decodes only, ferrox-server/src/batch_scheduler.rs:158-315;
its private loop can cut a prompt into chunks, generate.rs:152-186.)

Pages are taken per step, not reserved for the worst case at admission as the
reference does (generate.rs:44-80).  When a running request cannot get the pages
for its next tokens, the youngest running request is preempted: its pages and
slot are given back and it returns to the front of the waiting queue with
prompt := prompt + generated so far, to be recomputed; its sampler state stays,
so its continuation is the same.  The only running request is never preempted:
if it cannot grow, it is finished with reason "cache_full".

Order of a request's life, as in the reference (batch_scheduler.rs:195-237):
logits of its last position are sampled; EOS finishes it ("stop") without being
appended; otherwise the token is appended; reaching max_new_tokens or the
context limit finishes it ("length") without a forward pass for the last token.

A step's sampled ids may be read one step late, so that the next step is launched
while this one still runs: `commit_launched` advances the requests with a stand-in
(`UNKNOWN`) for each sampled token, which the next step takes from the device;
`resolve` puts the ids in once the host has them and finishes the requests whose
token was EOS (their part of the step launched meanwhile is thrown away).  What a
request generates is the same either way.  Before it preempts or gives up on a
request the scheduler calls `settle`, so such decisions are made on known tokens.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field

from ..sampling.sampler import SamplingParams, XorShift64

UNKNOWN = -1          # in `Request.generated`: a token that is sampled but not read back yet


@dataclass
class Request:
    id: object
    prompt: list
    max_new_tokens: int
    params: SamplingParams = field(default_factory=SamplingParams)
    eos_token_id: object = None       # None, one token id, or several: each of them ends the request
    ignore_eos: bool = False
    # progress
    generated: list = field(default_factory=list)
    n_computed: int = 0               # positions of prompt + generated already in the cache
    status: str = "waiting"           # waiting | running | finished
    finish_reason: str | None = None
    n_preempted: int = 0
    arrival: int = 0
    rng: XorShift64 = None

    def __post_init__(self):
        if self.rng is None:
            self.rng = XorShift64(self.params.seed)
        eos = self.eos_token_id
        self.stop_ids = frozenset() if eos is None else frozenset(
            int(t) for t in (eos if isinstance(eos, (list, tuple, set, frozenset)) else (eos,)))

    @property
    def tokens(self) -> list:
        return self.prompt + self.generated

    @property
    def n_pending(self) -> int:
        return len(self.prompt) + len(self.generated) - self.n_computed


@dataclass
class Scheduled:
    request: Request
    n_tokens: int
    samples: bool          # the portion reaches the request's last token: its logits are sampled
    place: int = -1        # where in `request.generated` the sampled token goes (set by `commit_launched`)


class Scheduler:
    def __init__(self, cache, *, max_tokens_per_step: int = 4096, prefill_chunk: int = 4096,
                 max_seqs: int | None = None, context_limit: int | None = None, vocab_size: int | None = None):
        """`cache` offers admit(id) -> bool, reserve(id, n) -> bool, release(id)."""
        if max_tokens_per_step < 1 or prefill_chunk < 1:
            raise ValueError("max_tokens_per_step and prefill_chunk must be >= 1")
        self.cache = cache
        self.max_tokens_per_step = max_tokens_per_step
        self.prefill_chunk = prefill_chunk
        self.max_seqs = max_seqs
        self.context_limit = context_limit
        self.vocab_size = vocab_size
        self.waiting: deque = deque()
        self.running: list = []
        self.finished: list = []
        self._arrivals = 0
        self.n_preemptions = 0
        self.settle = None        # callable -> bool: read the ids still in flight and `resolve` them; True if any were

    # ---- arrival -----------------------------------------------------------
    def add(self, req: Request) -> None:
        if not req.prompt:
            raise ValueError(f"request {req.id!r}: empty prompt")
        if self.vocab_size is not None:
            for t in req.prompt:
                if not 0 <= int(t) < self.vocab_size:        # ferrox-server/src/batch_scheduler.rs:271-279
                    raise ValueError(f"request {req.id!r}: token id {t} is outside the vocabulary of {self.vocab_size}")
        if self.context_limit is not None and len(req.prompt) >= self.context_limit:   # ferrox-cli/src/run.rs:602-607
            raise ValueError(f"request {req.id!r}: prompt of {len(req.prompt)} tokens does not fit the context "
                             f"of {self.context_limit}")
        req.arrival = self._arrivals
        self._arrivals += 1
        if req.max_new_tokens <= 0:
            self._finish(req, "length")
            return
        self.waiting.append(req)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ---- one step ------------------------------------------------------------
    def schedule(self) -> list:
        budget = self.max_tokens_per_step
        out: list = []
        scheduled_ids = set()
        # running requests, oldest first; decodes (one pending token) before prompt portions
        order = sorted(self.running, key=lambda r: (r.n_pending > 1, r.arrival))
        for req in order:
            if req.status != "running" or budget <= 0:
                continue
            n = min(req.n_pending, budget, self.prefill_chunk if req.n_pending > 1 else 1)
            while not self.cache.reserve(req.id, n):
                if self.settle is not None and self.settle():
                    # ids that were in flight are known now: a request may have ended and given pages back
                    if req.status != "running":
                        n = 0
                        break
                    continue
                victim = self._youngest_running(exclude=scheduled_ids)
                if victim is None or victim is req:
                    if len(self.running) == 1 or victim is None:
                        self._finish(req, "cache_full")
                    else:
                        self._preempt(req)
                    n = 0
                    break
                self._preempt(victim)
            if n:
                out.append(Scheduled(req, n, n == req.n_pending))
                scheduled_ids.add(req.id)
                budget -= n
        # admissions, first come first served; never preempt for them
        while self.waiting and budget > 0:
            if self.max_seqs is not None and len(self.running) >= self.max_seqs:
                break
            req = self.waiting[0]
            n = min(req.n_pending, budget, self.prefill_chunk)
            if not self.cache.admit(req.id):
                break
            if not self.cache.reserve(req.id, n):
                self.cache.release(req.id)
                if self.settle is not None and self.settle():
                    continue
                if not self.running:          # nothing will ever free pages for it
                    self.waiting.popleft()
                    self._finish(req, "cache_full")
                    continue
                break
            self.waiting.popleft()
            req.status = "running"
            self.running.append(req)
            out.append(Scheduled(req, n, n == req.n_pending))
            budget -= n
        # a request that `settle` ended after it was put on the list holds no pages any more
        return [s for s in out if s.request.status == "running"]

    def step_tokens(self, s: Scheduled) -> list:
        toks = s.request.tokens
        return toks[s.request.n_computed:s.request.n_computed + s.n_tokens]

    def commit(self, scheduled: list, sampled: dict) -> None:
        """After the step: advance every scheduled request; `sampled[id]` is the token drawn from
        the logits of a request whose portion reached its end."""
        self.commit_launched(scheduled)
        self.resolve(scheduled, sampled)

    def commit_launched(self, scheduled: list) -> None:
        """The step is launched: advance every scheduled request that is still running, with `UNKNOWN` in the
        place of each sampled token.  Whether a request ends for its length does not depend on the token."""
        for s in scheduled:
            req = s.request
            if req.status != "running":          # ended by an id that was read after the step was put together
                s.samples = False
                continue
            req.n_computed += s.n_tokens
            if not s.samples:
                continue
            s.place = len(req.generated)
            req.generated.append(UNKNOWN)
            if len(req.generated) >= req.max_new_tokens:
                self._finish(req, "length")
            elif self.context_limit is not None and len(req.prompt) + len(req.generated) >= self.context_limit:
                self._finish(req, "length")

    def resolve(self, scheduled: list, sampled: dict) -> None:
        """The ids of a step that `commit_launched` advanced are known: `sampled[id]` for every request it
        sampled.  EOS ends the request without being appended, also where its length ended it already."""
        for s in scheduled:
            if not s.samples:
                continue
            req, tok = s.request, int(sampled[s.request.id])
            if req.generated[s.place] != UNKNOWN:
                raise RuntimeError(f"request {req.id!r}: token {s.place} was resolved twice")
            if tok in req.stop_ids and not req.ignore_eos:
                del req.generated[s.place:]
                if req.status == "waiting":          # preempted meanwhile
                    self.waiting.remove(req)
                if req.status == "finished":
                    req.finish_reason = "stop"
                else:
                    self._finish(req, "stop")
            else:
                req.generated[s.place] = tok

    # ---- internals -----------------------------------------------------------
    def _youngest_running(self, exclude=()):
        cands = [r for r in self.running if r.id not in exclude]
        return max(cands, key=lambda r: r.arrival) if cands else None

    def _preempt(self, req: Request) -> None:
        self.cache.release(req.id)
        self.running.remove(req)
        req.status = "waiting"
        req.n_computed = 0
        req.n_preempted += 1
        self.n_preemptions += 1
        self.waiting.appendleft(req)

    def _finish(self, req: Request, reason: str) -> None:
        if req.status == "running":
            self.cache.release(req.id)
            self.running.remove(req)
        req.status = "finished"
        req.finish_reason = reason
        self.finished.append(req)
