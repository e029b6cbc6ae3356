"""The Python entry point: an `Engine` over one model on one GPU.

    engine = Engine("/path/to/model")                      # config.json + safetensors
    engine = Engine(config=cfg_dict, random_weights=0)     # seeded random weights, no files
    ids = engine.generate([[1, 2, 3]], max_new_tokens=16, temperature=0.0)

Generation follows the reference's loop (ferrox-cli/src/run.rs:651-676,
ferrox-server/src/batch_scheduler.rs:158-243): prefill, then sample -> append ->
forward until EOS, the token limit or the context limit; here all requests share
one continuously batched step.  The host runs one step ahead of the GPU: a step is
launched with the tokens that the step before it sampled still on the device, and
those ids are read while it runs (`Engine.overlap_steps`).
"""
from __future__ import annotations

import time
from dataclasses import dataclass

import torch

from ..sampling.sampler import SamplingParams, launch_sample_rows
from .loading import load_model, parse_dtype, random_model
from .runner import ModelRunner, StepEntry
from .scheduler import UNKNOWN, Request, Scheduler


@dataclass
class Completion:
    token_ids: list
    finish_reason: str
    n_prompt_tokens: int
    n_preempted: int = 0


class Engine:
    def __init__(self, model_dir: str | None = None, *, config=None, random_weights: int | None = None,
                 model=None, dtype="bfloat16", device="cuda:0", block_size: int = 64, num_pages: int | None = None,
                 max_seqs: int = 64, max_tokens_per_step: int = 4096, prefill_chunk: int = 4096,
                 ctx_size: int = 0):
        """One of: `model_dir` (config.json + safetensors), `config` with `random_weights=<seed>`, or `model`,
        a model that is loaded already (its dtype and device are taken)."""
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU is visible; this engine has no CPU path")
        self.dtype = parse_dtype(dtype)
        if model is not None:
            self.model, self.dtype = model, model.act_dtype
        elif model_dir is not None:
            self.model = load_model(model_dir, self.dtype, device)
        elif config is not None and random_weights is not None:
            self.model = random_model(config, int(random_weights), self.dtype, device)
        else:
            raise ValueError("give a model folder, or a configuration together with random_weights=<seed>")
        spec = self.model.spec
        self.context_limit = ctx_size if ctx_size > 0 else spec.max_positions      # run.rs:551-559
        if num_pages is None:        # room for max_seqs requests of half the context each, at least one full
            num_pages = max(-(-self.context_limit // block_size) + 1,
                            max_seqs * (-(-self.context_limit // block_size)) // 2)
        self.runner = ModelRunner(self.model, block_size=block_size, num_pages=num_pages, max_seqs=max_seqs)
        self.max_seqs = max_seqs
        self.max_tokens_per_step = max_tokens_per_step
        self.prefill_chunk = prefill_chunk
        self.eos_token_id = spec.eos_token_id
        self.last_stats: dict = {}
        self.overlap_steps = True    # False: every step's ids are read before the next step is put together
        self.time_steps = False      # True: every step is bracketed by events and last_stats also says where the time went

    @property
    def vocab_size(self) -> int:
        return self.model.spec.vocab_size

    def step(self, entries: list):
        """Direct access to the step function (entries are `StepEntry`s whose pages are reserved)."""
        return self.runner.step(entries)

    def generate(self, prompts: list, max_new_tokens: int = 128, temperature: float = 0.0, top_k: int = 0,
                 top_p: float = 1.0, repetition_penalty: float = 1.0, presence_penalty: float = 0.0,
                 frequency_penalty: float = 0.0, seed: int = 0, ignore_eos: bool = False,
                 eos_token_id=None) -> list:
        """Token ids generated for each prompt (a list of token ids), in order.  `eos_token_id`: one id or a list
        of ids that end a request (default: the model's own, which may be several)."""
        return [c.token_ids for c in self.generate_detailed(
            prompts, max_new_tokens, SamplingParams(temperature, top_k, top_p, repetition_penalty,
                                                    presence_penalty, frequency_penalty, seed),
            ignore_eos=ignore_eos, eos_token_id=eos_token_id)]

    def generate_detailed(self, prompts: list, max_new_tokens, params: SamplingParams | list | None = None,
                          ignore_eos: bool = False, eos_token_id=None, on_token=None) -> list:
        """`params` may be one `SamplingParams` for all or one per prompt; `max_new_tokens` likewise.
        Request i draws from a generator seeded with its own params.seed.  `on_token(i, token)` is called for
        every token that request i generates, in order, as soon as the host has read it (the reference prints
        as it generates, ferrox-cli/src/run.rs:651-676)."""
        eos = eos_token_id if eos_token_id is not None else self.eos_token_id
        sched = Scheduler(self.runner, max_tokens_per_step=self.max_tokens_per_step,
                          prefill_chunk=self.prefill_chunk, max_seqs=self.max_seqs,
                          context_limit=self.context_limit, vocab_size=self.vocab_size)
        reqs = []
        for i, p in enumerate(prompts):
            sp = params[i] if isinstance(params, (list, tuple)) else (params or SamplingParams())
            mx = max_new_tokens[i] if isinstance(max_new_tokens, (list, tuple)) else max_new_tokens
            if mx < 0:                                   # -1: fill the context (run.rs:609-614)
                mx = self.context_limit - len(p)
            mx = min(mx, self.context_limit - len(p))
            r = Request(i, [int(t) for t in p], mx, SamplingParams(**vars(sp)), eos, ignore_eos)
            reqs.append(r)
            sched.add(r)
        t0 = time.time()
        n_steps = n_tokens = 0
        marks = []            # per step: [event at its first device operation, event after its last launch, all decodes?]
        launching = 0.0       # (time_steps) seconds the host spent putting steps together and launching them
        if self.time_steps:
            self.runner.before_launch = lambda: marks[-1][0].record()
        # the step whose sampled ids the host has not read yet: its batch, the requests of the rows, the ids on
        # the device, their copy in pinned memory and the event after that copy
        inflight = None
        told = [0] * len(reqs)        # how many of each request's tokens `on_token` has been given

        def settle() -> bool:
            nonlocal inflight
            if inflight is None:
                return False
            batch, rows, _, host_ids, copied = inflight
            inflight = None
            copied.synchronize()
            sched.resolve(batch, {r.id: t for r, t in zip(rows, host_ids.tolist())})
            if on_token is not None:
                for r in rows:           # a request's tokens that became known (an EOS is never among them)
                    while told[r.id] < len(r.generated) and r.generated[told[r.id]] != UNKNOWN:
                        on_token(r.id, r.generated[told[r.id]])
                        told[r.id] += 1
            return True

        sched.settle = settle
        try:
            while True:
                batch = sched.schedule() if sched.has_work() else []
                if not batch:
                    if settle():              # the last ids may end a request and free what another waits for
                        continue
                    if sched.has_work():
                        raise RuntimeError("scheduler made no progress")
                    break
                row_of = {r.id: i for i, r in enumerate(inflight[1])} if inflight is not None else {}
                entries, pairs, first = [], [], 0
                for s in batch:
                    toks = sched.step_tokens(s)
                    if toks[-1] == UNKNOWN:         # sampled by the step in flight: taken from the device
                        pairs.append((first + len(toks) - 1, row_of[s.request.id]))
                        toks[-1] = 0
                    entries.append(StepEntry(s.request.id, toks, [s.n_tokens - 1] if s.samples else []))
                    first += len(toks)
                if self.time_steps:
                    marks.append([torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True),
                                  all(s.n_tokens == 1 for s in batch)])
                    t_launch = time.perf_counter()
                logits = self.runner.step(entries, feed=(inflight[2], pairs) if pairs else None)
                rows = [s.request for s in batch if s.samples]
                launched = None
                if rows:
                    ids = launch_sample_rows(logits, [r.params for r in rows], [r.rng for r in rows],
                                             [r.generated for r in rows])
                    host_ids = torch.empty(len(rows), dtype=torch.int32, pin_memory=True)
                    host_ids.copy_(ids, non_blocking=True)
                    copied = torch.cuda.Event()
                    copied.record()
                    launched = (batch, rows, ids, host_ids, copied)
                if self.time_steps:
                    marks[-1][1].record()
                    launching += time.perf_counter() - t_launch
                settle()                      # the ids of the step before this one: they come while this one runs
                sched.commit_launched(batch)
                inflight = launched
                if not self.overlap_steps or any(r.params.uses_history for r in rows):
                    settle()                  # penalties over what was generated need every token on the host
                n_steps += 1
                n_tokens += sum(s.n_tokens for s in batch)
        finally:
            self.runner.before_launch = None
            for r in list(sched.running):
                self.runner.release(r.id)
        self.last_stats = {"steps": n_steps, "tokens": n_tokens, "seconds": time.time() - t0,
                           "preemptions": sched.n_preemptions}
        if self.time_steps and marks:
            # from a step's first device operation to the end of its last kernel, as the GPU saw it; between the
            # end of one step and the first operation of the next the GPU waits for the host (reading the ids
            # back, scheduling, packing): `host_gap_seconds`.  Waits inside a step (kernels launched one by one
            # faster than they are submitted) are not seen this way.
            torch.cuda.synchronize()
            spans = [a.elapsed_time(b) * 1e-3 for a, b, _ in marks]
            gaps = [marks[i][1].elapsed_time(marks[i + 1][0]) * 1e-3 for i in range(len(marks) - 1)]
            dec = [i for i, m in enumerate(marks) if m[2]]
            # `launch_seconds`: what the host spent inside the steps (packing, one launch after the other, the sampling
            # call); where it comes near `gpu_seconds` the kernels of a step wait for their launches.
            self.last_stats.update(gpu_seconds=sum(spans), host_gap_seconds=sum(gaps), decode_steps=len(dec),
                                   launch_seconds=launching,
                                   decode_gpu_seconds=sum(spans[i] for i in dec),
                                   decode_gap_seconds=sum(gaps[i - 1] for i in dec if i > 0))
        return [Completion(r.generated, r.finish_reason or "aborted", len(r.prompt), r.n_preempted) for r in reqs]


def generate(model_dir: str, prompts: list, **kw) -> list:
    """One-call form: load the model folder, generate, return the token ids."""
    engine_kw = {k: kw.pop(k) for k in ("dtype", "device", "block_size", "num_pages", "max_seqs",
                                        "max_tokens_per_step", "prefill_chunk", "ctx_size") if k in kw}
    return Engine(model_dir, **engine_kw).generate(prompts, **kw)
