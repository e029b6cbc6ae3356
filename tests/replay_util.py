"""Shared by the GPU tests: traces that cut the same requests in different ways,
a driver that runs them through the engine's step function, and the comparison
with the plain implementation."""
from __future__ import annotations

import functools
import random

import torch

import plain_qwen2moe as plain


def make_requests(vocab: int, lengths, seed: int) -> dict:
    rng = random.Random(seed)
    return {f"r{i}": [rng.randrange(vocab) for _ in range(n)] for i, n in enumerate(lengths)}


# ---- the four ways of cutting ------------------------------------------------
def trace_whole(requests: dict) -> list:
    steps = []
    for rid, toks in requests.items():
        steps.append({"entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]})
    return steps


def trace_tail_decode(requests: dict, tail: int = 32) -> list:
    steps = []
    for rid, toks in requests.items():
        head = max(0, len(toks) - tail)
        if head:
            steps.append({"entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}], "end": []})
        for i in range(head, len(toks)):
            steps.append({"entries": [{"id": rid, "tokens": [toks[i]], "want": [0]}],
                          "end": [rid] if i == len(toks) - 1 else []})
    return steps


def trace_portions(requests: dict, sizes=(7, 5, 3, 2, 11, 2, 16, 9, 2, 4)) -> list:
    steps, k = [], 0
    for rid, toks in requests.items():
        pos = 0
        while pos < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - pos)
            if len(toks) - pos - n == 1:       # never leave a portion of one token behind... take it along
                n += 1
            k += 1
            steps.append({"entries": [{"id": rid, "tokens": toks[pos:pos + n], "want": list(range(n))}],
                          "end": [rid] if pos + n == len(toks) else []})
            pos += n
    return steps


def trace_mixed(requests: dict, seed: int, max_live: int = 4, decode_tail: int = 12) -> list:
    """Up to `max_live` requests at a time; each goes through its tokens in portions of random
    size and its last `decode_tail` tokens one by one; a request may sit a step out."""
    rng = random.Random(seed)
    todo = list(requests.items())
    live: dict = {}
    steps = []
    while todo or live:
        while todo and len(live) < max_live:
            rid, toks = todo.pop(0)
            live[rid] = [toks, 0]
        entries, end = [], []
        for rid, (toks, pos) in list(live.items()):
            if len(live) > 1 and rng.random() < 0.2:
                continue                                   # left out of this step, goes on later
            left = len(toks) - pos
            if left <= decode_tail:
                n = 1
            else:
                n = min(rng.choice([2, 3, 5, 8, 13, 24]), left - decode_tail)
                if n == 1:
                    n = 1
            entries.append({"id": rid, "tokens": toks[pos:pos + n], "want": list(range(n))})
            live[rid][1] = pos + n
            if pos + n == len(toks):
                end.append(rid)
                del live[rid]
        if entries:
            steps.append({"entries": entries, "end": end})
    return steps


def max_live_tokens(steps: list, round_to: int = 64) -> int:
    """The most tokens live requests hold at any time, each rounded up to `round_to`."""
    held: dict = {}
    peak = 0
    for st in steps:
        for e in st["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(-(-n // round_to) * round_to for n in held.values()))
        for rid in st["end"]:
            held.pop(rid, None)
    return peak


# ---- running a trace through the engine ---------------------------------------
def run_trace(runner, steps: list, routing: dict | None = None) -> dict:
    """(request id, position) -> float32 logits row (CPU).  If `routing` is a dict it receives
    (request id, position) -> experts chosen in each sparse layer (the step then runs eagerly)."""
    from ferrox_amd.engine.runner import StepEntry
    from ferrox_amd.parts.moe import SparseMoE
    out, pos = {}, {}
    graphs = runner.use_graphs
    if routing is not None:
        runner.use_graphs = False
    for st in steps:
        entries = []
        for e in st["entries"]:
            rid = e["id"]
            if rid not in runner.manager:
                assert runner.admit(rid), f"no slot for {rid}"
                pos[rid] = 0
            assert runner.reserve(rid, len(e["tokens"])), f"out of pages for {rid}"
            entries.append(StepEntry(rid, e["tokens"], e["want"]))
        if routing is not None:
            SparseMoE.record = []
        logits = runner.step(entries)
        if routing is not None:
            per_layer = [t.cpu().tolist() for t in SparseMoE.record]      # [sparse layer][token][slot]
            SparseMoE.record = None
            tok = 0
            for e in st["entries"]:
                for i in range(len(e["tokens"])):
                    routing[(e["id"], pos[e["id"]] + i)] = [layer[tok] for layer in per_layer]
                    tok += 1
        runner.manager.check_invariants()
        row = 0
        if logits is not None:
            logits = logits.float().cpu()
        for e in st["entries"]:
            for w in e["want"]:
                out[(e["id"], pos[e["id"]] + w)] = logits[row]
                row += 1
            pos[e["id"]] += len(e["tokens"])
        for rid in st["end"]:
            runner.release(rid)
            pos.pop(rid, None)
    runner.use_graphs = graphs
    return out


@functools.lru_cache(maxsize=None)
def _plain_model(folder: str):
    return plain.load_folder(folder)


_plain_cache: dict = {}


def plain_logits(folder: str, tokens, with_margins: bool = False):
    """logits [T, V] of the plain model (and, on request, its router margins and choices)"""
    key = (folder, tuple(tokens))
    if key not in _plain_cache:
        cfg, w = _plain_model(folder)
        margins, chosen = [], []
        _plain_cache[key] = (plain.forward(cfg, w, list(tokens), margins=margins, chosen=chosen), margins, chosen)
    return _plain_cache[key] if with_margins else _plain_cache[key][0]


def same_choice(a, b) -> bool:
    """the same experts in every sparse layer; their order only decides the order of a sum"""
    return len(a) == len(b) and all(sorted(x) == sorted(y) for x, y in zip(a, b))


def compare(got: dict, folder: str, requests: dict, atol: float, rtol: float, what: str,
            routing: dict | None = None, flip_margin: float = 0.05, stol: float = 0.0) -> float:
    """Every (request, position) of `got` against the plain implementation; returns the largest error.

    `routing` (bfloat16 only): the experts the engine chose.  Rounding may flip a choice where two
    router probabilities nearly tie.  Where the engine's choice differs from the plain model's, the
    tie must be a near one (relative gap below `flip_margin`), and the plain model is then run with
    the engine's choice, so that everything else is still compared at every position.
    The bound on an element is atol + rtol * |plain| + stol * (standard deviation of the plain
    logits of that position)."""
    worst, worst_at, flips, total = 0.0, None, 0, 0
    for rid, toks in requests.items():
        ref, margins, chosen = plain_logits(folder, toks, with_margins=True)
        if routing is not None:
            mine = [routing[(rid, p)] for p in range(len(toks))]
            differ = [p for p in range(len(toks)) if not same_choice(mine[p], chosen[p])]
            for p in differ:
                assert margins[p] < flip_margin, (f"{what}: request {rid} position {p}: the engine chose experts "
                                                  f"{mine[p]}, the plain model {chosen[p]} with a margin of {margins[p]:.3f}")
            if differ:
                flips += len(differ)
                cfg, w = _plain_model(folder)
                ref = plain.forward(cfg, w, list(toks), routing=mine)
        for p in range(len(toks)):
            assert (rid, p) in got, f"{what}: no logits for request {rid} position {p}"
            g = got[(rid, p)].double()
            assert torch.isfinite(g).all(), f"{what}: non-finite logits for {rid} position {p}"
            total += 1
            err = (g - ref[p]).abs()
            bound = atol + rtol * ref[p].abs() + stol * float(ref[p].std())
            if (err > bound).any():
                i = int((err - bound).argmax())
                raise AssertionError(f"{what}: request {rid} position {p} vocab {i}: engine {float(g[i]):.7f}, "
                                     f"plain {float(ref[p][i]):.7f}, |diff| {float(err[i]):.3e} > {float(bound[i]):.3e}")
            if float(err.max()) > worst:
                worst, worst_at = float(err.max()), (rid, p)
    # a flip is only accepted above where the plain model's own margin is below `flip_margin`; their
    # share must stay small (one position is the least a short trace can show)
    assert flips <= max(1, 0.1 * total), f"{what}: {flips} of {total} positions were routed differently"
    print(f"[{what}] largest |engine - plain| = {worst:.3e} at {worst_at}; {flips}/{total} positions routed on a near-tie")
    return worst
