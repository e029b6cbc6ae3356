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
    (request id, position) -> experts chosen in each sparse layer, read from the engine's routing
    trace (recorded decode steps are replayed as always: the trace's copies are part of them)."""
    import contextlib
    from ferrox_amd import debug
    from ferrox_amd.engine.runner import StepEntry
    out, pos = {}, {}
    with (debug.trace_routing() if routing is not None else contextlib.nullcontext()) as trace:
        for st in steps:
            entries = []
            for e in st["entries"]:
                rid = e["id"]
                if rid not in runner.manager:
                    assert runner.admit(rid), f"no slot for {rid}"
                    pos[rid] = 0
                assert runner.reserve(rid, len(e["tokens"])), f"out of pages for {rid}"
                entries.append(StepEntry(rid, e["tokens"], e["want"]))
            logits = runner.step(entries)
            if routing is not None:
                per_layer = trace.read()                                  # [sparse layer][token][slot]
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


_float32_cache: dict = {}


def float32_noise(folder: str, tokens) -> float:
    """The largest deviation, over all logits of the sequence, of the plain model worked out in float32 (the same
    formulas, the library's float32 arithmetic on the CPU) from the plain model in float64: what float32 rounding
    does to this model on these tokens."""
    key = (folder, tuple(tokens))
    if key not in _float32_cache:
        cfg, w = plain.load_folder(folder, dtype=torch.float32)
        low = plain.forward(cfg, w, list(tokens), dtype=torch.float32).double()
        _float32_cache[key] = float((low - plain_logits(folder, tokens)).abs().max())
    return _float32_cache[key]


_stored_cache: dict = {}


def stored_logits(folder: str, tokens, routing, with_probs: bool = False):
    """logits [T, V] of the plain model that rounds to bfloat16 where activations are stored, with the
    experts of `routing` (and, on request, its router's probabilities [position][sparse layer][expert])"""
    key = (folder, tuple(tokens), repr(routing))
    if key not in _stored_cache:
        cfg, w = _plain_model(folder)
        probs = []
        _stored_cache[key] = (plain.forward(cfg, w, list(tokens), routing=routing, stored=plain.to_bfloat16,
                                            router_probs=probs), probs)
    return _stored_cache[key] if with_probs else _stored_cache[key][0]


def same_choice(a, b) -> bool:
    """the same experts in every sparse layer; their order only decides the order of a sum"""
    return len(a) == len(b) and all(sorted(x) == sorted(y) for x, y in zip(a, b))


def near_tie_choice(chosen, probs, margin: float) -> bool:
    """Whether `chosen` is a top-k of `probs` up to a relative perturbation of `margin`: no expert that
    was left out has a probability more than `margin` above the smallest one that was taken."""
    taken = set(chosen)
    if len(taken) != len(chosen) or not all(0 <= e < len(probs) for e in taken):
        return False
    low = min(probs[e] for e in taken)
    left_out = [p for e, p in enumerate(probs) if e not in taken]
    return not left_out or low >= (1.0 - margin) * max(left_out)


# How the bfloat16 engine is measured.  `plain.forward(..., stored=plain.to_bfloat16)` is the plain model with
# rounding at exactly the places where an engine with bfloat16 activations stores a tensor (float64 otherwise).
# Its deviation from the plain model says what those roundings alone do to this model's logits on these tokens:
# noise on every logit, r = pooled rms((model - plain) / sigma_row) and r_row the same for one row (rows that see
# few keys are noisier than the pool), and now and then much more on one logit that the model is sensitive at
# (under a tied head the current token's own logit, ten spreads out, moves by 6 % of a spread where an attention
# of one narrow head leaves few terms to average over).  The engine is held against that rounding model.  Where
# it rounds the very numbers that the model rounds (prompt portions: a norm, then a product) it shares most of the
# model's deviation; where it rounds other numbers of the same size (few tokens: the norm's scale is applied
# behind the product, so x * w is rounded instead of x * s * w) its roundings are independent of the model's, and
# engine - model is the difference of two independent draws of the same noise, sqrt(2) r.  This is a model of
# rounding, measured on the model and the tokens at hand, not a derivation from first principles; its three
# limits follow from one constant:
#   * pooled: rms((engine - model) / sigma_row) <= RMS_FACTOR * r, RMS_FACTOR = 1.5 (sqrt(2), and a margin);
#   * every row: rms over the row's logits <= ROW_FACTOR * max(r, r_row) (a row's own noise is known from one
#     draw only, and a row that is off as a whole, a missed page or chunk of keys, is off by far more);
#   * every logit: |engine - model| <= peak(N) * RMS_FACTOR * max(r, r_row) * sigma_row, where peak(N) =
#     1.25 * sqrt(2 ln N): the largest of the N compared logits lies near sqrt(2 ln N) deviations if they are
#     Gaussian (4.7 for 5e4 logits, 5.3 for a million), and a margin of a quarter; what the pooled limit allows
#     on average must be allowed at the peak.  (An earlier form had 7 in place of peak(N) * RMS_FACTOR, which is
#     8.7 for 5e4 logits and 9.9 for a million: it took the engine's noise for r itself, and a sequence of 2,100
#     tokens, 8e5 logits whose roundings are independent of the model's, reached 1.01 of it.)
# Outlier logits (more than OUTLIER spreads from zero) are coherent sums, to which a relative shift of the
# sublayers' output against the embedding passes undiminished; there the model's and the engine's roundings need
# not agree (seen: model +0.34 %, engine +0.07 % of a logit 17 spreads out).  For them the bound grows by
# OUTLIER_FACTOR * rel * |logit|, rel being the largest relative deviation from the plain model that the rounding
# model shows on any outlier of the comparison (0.3-0.7 % where there are outliers at all).
RMS_FACTOR, ROW_FACTOR, OUTLIER, OUTLIER_FACTOR = 1.5, 3.0, 5.0, 1.5


def peak(n: int) -> float:
    """where the largest of n Gaussian deviations lies, in standard deviations, with a margin of a quarter"""
    import math
    return 1.25 * math.sqrt(2.0 * math.log(max(n, 2)))


def compare(got: dict, folder: str, requests: dict, atol: float, rtol: float, what: str,
            routing: dict | None = None, flip_margin: float = 0.05, storage: str | None = None,
            noise_factor: float = 0.0) -> float:
    """Every (request, position) of `got` against the plain implementation; returns the largest error.

    `routing` (bfloat16 only): the experts the engine chose.  Rounding may flip a choice where two
    router probabilities nearly tie.  Where the engine's choices differ from the plain model's, the
    plain model is run again with the engine's choices (so that everything else is still compared at
    every position, and later layers see what the engine saw), and every choice of that sequence, in
    every sparse layer, must be a top-k of the plain router's probabilities up to a relative
    perturbation of `flip_margin`: an expert is only ever exchanged for one whose probability is
    within that margin.  (With `storage`, a choice also passes if it is such a top-k of the probabilities of the
    rounding model's router: where rounding at the stored tensors alone moves two probabilities past each other
    by more than the margin, which models made sensitive on purpose show, the engine may follow it.)
    Without `storage` the bound on an element is atol + rtol * |plain|, plus `noise_factor` times the request's
    `float32_noise` (for models that are made sensitive on purpose, where a float32 evaluation of the plain
    formulas itself leaves the fixed bound).  With storage="bfloat16" the bounds
    are what the rounding model above gives for this model and these tokens (atol and rtol are not used)."""
    worst, worst_at, flips, total = 0.0, None, 0, 0
    rows = []          # (request, position, plain logits, rounding model's logits or None)
    for rid, toks in requests.items():
        ref, margins, chosen = plain_logits(folder, toks, with_margins=True)
        mine = chosen
        if routing is not None:
            mine = [routing[(rid, p)] for p in range(len(toks))]
            differ = [p for p in range(len(toks)) if not same_choice(mine[p], chosen[p])]
            if differ:
                flips += len(differ)
                cfg, w = _plain_model(folder)
                probs = []
                ref = plain.forward(cfg, w, list(toks), routing=mine, router_probs=probs)
                for p in range(len(toks)):
                    for j, ids in enumerate(mine[p]):
                        if near_tie_choice(ids, probs[p][j], flip_margin):
                            continue
                        rounded = stored_logits(folder, toks, mine, with_probs=True)[1] if storage is not None else None
                        assert rounded is not None and near_tie_choice(ids, rounded[p][j], flip_margin), (
                            f"{what}: request {rid} position {p} sparse layer {j}: the engine chose experts {ids}, "
                            f"the plain router's probabilities are {[round(x, 5) for x in probs[p][j]]}"
                            + (f", the rounding model's {[round(x, 5) for x in rounded[p][j]]}" if rounded else ""))
            else:
                mine = chosen
        model = None
        if storage is not None:
            assert storage == "bfloat16"
            model = stored_logits(folder, toks, mine)
        for p in range(len(toks)):
            assert (rid, p) in got, f"{what}: no logits for request {rid} position {p}"
            rows.append((rid, p, ref[p], model[p] if model is not None else None))
    slack = {rid: noise_factor * float32_noise(folder, toks) for rid, toks in requests.items()} if noise_factor else {}
    r, rel, noise_rows = 0.0, 0.0, []
    if storage is not None:
        noise_rows = [float(((m - ref) / ref.std()).pow(2).mean()) for _, _, ref, m in rows]
        r = (sum(noise_rows) / len(noise_rows)) ** 0.5
        for _, _, ref, m in rows:
            far = ref.abs() > OUTLIER * ref.std()
            if far.any():
                rel = max(rel, float(((m - ref).abs() / ref.abs())[far].max()))
    mine_sq, n_elems = 0.0, 0
    sigmas = peak(sum(ref.numel() for _, _, ref, _ in rows)) * RMS_FACTOR
    worst_row = 0.0
    for k, (rid, p, ref, model_row) in enumerate(rows):
        g = got[(rid, p)].double()
        assert torch.isfinite(g).all(), f"{what}: non-finite logits for {rid} position {p}"
        total += 1
        if storage is None:
            err = (g - ref).abs()
            bound = atol + rtol * ref.abs() + slack.get(rid, 0.0)
        else:
            err = (g - model_row).abs()
            noise = max(r, noise_rows[k] ** 0.5)
            bound = torch.full_like(err, sigmas * noise * float(ref.std()))
            far = ref.abs() > OUTLIER * ref.std()
            bound = bound + OUTLIER_FACTOR * rel * ref.abs() * far
            mine_sq += float((err / ref.std()).pow(2).sum())
            n_elems += err.numel()
            # the row as a whole, outliers aside (their bound is their own)
            row_rms = float((err[~far] / ref.std()).pow(2).mean().sqrt()) if (~far).any() else 0.0
            worst_row = max(worst_row, row_rms / noise)
            assert row_rms <= ROW_FACTOR * noise, (
                f"{what}: request {rid} position {p}: the row deviates from the rounding model by {row_rms:.4f} spreads "
                f"(rms), rounding alone moves it by {noise:.4f}")
        if (err > bound).any():
            i = int((err - bound).argmax())
            other = f"rounding model {float(model_row[i]):.7f}, " if storage is not None else ""
            raise AssertionError(f"{what}: request {rid} position {p} vocab {i}: engine {float(g[i]):.7f}, {other}"
                                 f"plain {float(ref[i]):.7f}, |diff| {float(err[i]):.3e} > {float(bound[i]):.3e}")
        if float(err.max()) > worst:
            worst, worst_at = float(err.max()), (rid, p)
    note = ""
    if storage is not None:
        mine_rms = (mine_sq / max(1, n_elems)) ** 0.5
        note = (f"; rms/spread: engine - rounding model {mine_rms:.4f}, rounding model - plain {r:.4f}; the worst row "
                f"{worst_row:.2f} of its noise; per-logit limit {sigmas:.1f} noise deviations; outliers move "
                f"by up to {rel:.4f} of themselves in the rounding model")
        assert mine_rms <= RMS_FACTOR * r, (f"{what}: the engine deviates from the rounding model by {mine_rms:.4f} spreads "
                                            f"(rms); rounding at the stored tensors alone moves the logits by {r:.4f}")
    print(f"[{what}] largest |engine - {'rounding model' if storage else 'plain'}| = {worst:.3e} at {worst_at}; {flips}/{total} positions routed on a near-tie{note}")
    return worst
