"""The scheduler's decisions, with the real cache manager and no GPU."""
import pytest

from ferrox_amd.cache import CacheManager
from ferrox_amd.engine.scheduler import Request, Scheduler
from ferrox_amd.sampling import SamplingParams, XorShift64

FULL = ("full",)


class Cache:
    """What the scheduler needs of the runner: admit, reserve, release."""

    def __init__(self, pages, block_size=4, slots=8):
        self.m = CacheManager({FULL: None}, pages, block_size, slots)

    def admit(self, rid):
        return self.m.admit(rid) is not None

    def reserve(self, rid, n):
        return self.m.extend(rid, self.m.length(rid) + n)

    def release(self, rid):
        self.m.release(rid)


def run(sched, next_token=lambda req: 1, max_steps=10_000):
    """Drives the scheduler as the engine does; returns the list of steps [(id, n_tokens, samples)]."""
    steps = []
    while sched.has_work():
        batch = sched.schedule()
        assert batch or not sched.has_work()
        if not batch:
            break
        steps.append([(s.request.id, s.n_tokens, s.samples) for s in batch])
        for s in batch:                                       # the runner's own check: pages are there
            assert sched.cache.m.length(s.request.id) == s.request.n_computed + s.n_tokens
        sched.commit(batch, {s.request.id: next_token(s.request) for s in batch if s.samples})
        sched.cache.m.check_invariants()
        assert len(steps) < max_steps
    return steps


def test_prompt_is_cut_into_portions_under_the_budget():
    sched = Scheduler(Cache(64), max_tokens_per_step=10, prefill_chunk=6)
    sched.add(Request("a", list(range(20)), max_new_tokens=3))
    steps = run(sched)
    assert steps[:4] == [[("a", 6, False)], [("a", 6, False)], [("a", 6, False)], [("a", 2, True)]]
    assert steps[4:] == [[("a", 1, True)], [("a", 1, True)]]                 # no forward pass for the last token
    r = sched.finished[0]
    assert r.finish_reason == "length" and r.generated == [1, 1, 1] and sched.cache.m.n_free_pages() == 64


def test_decodes_ride_along_with_prompt_portions():
    sched = Scheduler(Cache(64), max_tokens_per_step=8, prefill_chunk=8)
    sched.add(Request("a", [1, 2, 3], max_new_tokens=10))
    first = sched.schedule()
    sched.commit(first, {"a": 5})
    sched.add(Request("b", list(range(20)), max_new_tokens=2))
    batch = sched.schedule()
    assert [(s.request.id, s.n_tokens) for s in batch] == [("a", 1), ("b", 7)]       # decode first, rest of the budget
    sched.commit(batch, {"a": 5})
    batch = sched.schedule()
    assert [(s.request.id, s.n_tokens, s.samples) for s in batch] == [("a", 1, True), ("b", 7, False)]


def test_admission_is_first_come_first_served_and_capped():
    sched = Scheduler(Cache(64, slots=2), max_tokens_per_step=100, prefill_chunk=100, max_seqs=2)
    for i in range(3):
        sched.add(Request(i, [1, 2], max_new_tokens=2))
    batch = sched.schedule()
    assert [s.request.id for s in batch] == [0, 1]                    # the third waits for a slot
    sched.commit(batch, {0: 1, 1: 1})
    run(sched)
    assert [r.id for r in sched.finished] == [0, 1, 2]


def test_eos_stops_without_being_appended_and_can_be_ignored():
    sched = Scheduler(Cache(64))
    sched.add(Request("a", [1, 2], max_new_tokens=5, eos_token_id=9))
    sched.add(Request("b", [1, 2], max_new_tokens=3, eos_token_id=9, ignore_eos=True))
    toks = iter([4, 4, 9, 9, 9, 9, 9])
    run(sched, lambda req: 9 if len(req.generated) >= 1 else 4)
    a, b = sorted(sched.finished, key=lambda r: r.id)
    assert (a.finish_reason, a.generated) == ("stop", [4]) and (b.finish_reason, b.generated) == ("length", [4, 9, 9])


def test_any_of_several_stop_ids_ends_a_request():
    """chat variants of this family stop on either of two ids (config.json gives a list)"""
    sched = Scheduler(Cache(64))
    sched.add(Request("a", [1, 2], max_new_tokens=9, eos_token_id=[9, 11]))
    sched.add(Request("b", [1, 2], max_new_tokens=9, eos_token_id=(11, 9)))
    sched.add(Request("c", [1, 2], max_new_tokens=4, eos_token_id=[9, 11], ignore_eos=True))
    sched.add(Request("d", [1, 2], max_new_tokens=4, eos_token_id=[]))            # no stop id at all
    picks = {"a": [4, 5, 11, 4], "b": [4, 9, 4, 4], "c": [9, 11, 4, 4], "d": [9, 11, 4, 4]}
    run(sched, lambda req: picks[req.id][len(req.generated)])
    by = {r.id: (r.finish_reason, r.generated) for r in sched.finished}
    assert by == {"a": ("stop", [4, 5]), "b": ("stop", [4]), "c": ("length", [9, 11, 4, 4]), "d": ("length", [9, 11, 4, 4])}


def test_bad_requests_are_refused():
    sched = Scheduler(Cache(8), context_limit=10, vocab_size=50)
    with pytest.raises(ValueError):
        sched.add(Request("e", [], 1))
    with pytest.raises(ValueError):
        sched.add(Request("v", [1, 50], 1))                     # id outside the vocabulary
    with pytest.raises(ValueError):
        sched.add(Request("l", list(range(10)), 1))             # prompt fills the context
    sched.add(Request("z", [1], max_new_tokens=0))
    assert sched.finished[0].finish_reason == "length" and not sched.has_work()
    sched.add(Request("c", [1] * 8, max_new_tokens=100))        # stops at the context limit
    run(sched)
    c = sched.finished[-1]
    assert c.finish_reason == "length" and len(c.prompt) + len(c.generated) == 10


def test_when_pages_run_out_the_youngest_is_preempted_and_recomputed():
    # 6 pages of 4: two requests with 8-token prompts fill 4 pages and grow until the pool is empty
    sched = Scheduler(Cache(6, block_size=4), max_tokens_per_step=64, prefill_chunk=64)
    sched.add(Request("old", list(range(8)), max_new_tokens=12))
    sched.add(Request("young", list(range(8)), max_new_tokens=12))
    counter = {"old": 100, "young": 200}

    def nxt(req):
        counter[req.id] += 1
        return counter[req.id]

    steps = run(sched, nxt)
    old, young = sorted(sched.finished, key=lambda r: r.id)
    assert sched.n_preemptions >= 1 and young.n_preempted >= 1 and old.n_preempted == 0
    assert old.finish_reason == young.finish_reason == "length"
    assert old.generated == list(range(101, 113)) and young.generated == list(range(201, 213))   # nothing lost or doubled
    # after its preemption the young request came back with prompt + generated as one portion
    assert any(rid == "young" and n > 8 for step in steps for rid, n, _ in step)
    assert sched.cache.m.n_free_pages() == 6 and sched.cache.m.slots.n_free == 8


def test_the_only_runner_is_never_preempted_but_ends_when_the_cache_is_full():
    sched = Scheduler(Cache(3, block_size=4), max_tokens_per_step=64, prefill_chunk=64)
    sched.add(Request("big", list(range(10)), max_new_tokens=50))
    run(sched)
    r = sched.finished[0]
    assert r.finish_reason == "cache_full" and len(r.prompt) + len(r.generated) == 13 and r.n_preempted == 0
    # a prompt that can never fit ends the same way instead of waiting for ever
    sched.add(Request("huge", list(range(40)), max_new_tokens=1))
    run(sched)
    assert sched.finished[-1].finish_reason == "cache_full" and sched.cache.m.n_free_pages() == 3


def test_each_request_has_its_own_seeded_generator():
    a, b = Request(1, [1], 4, SamplingParams(temperature=1.0, seed=7)), Request(2, [1], 4, SamplingParams(temperature=1.0, seed=7))
    xs = [a.rng.next_f32() for _ in range(3)]
    assert xs == [b.rng.next_f32() for _ in range(3)] == [XorShift64(7).next_f32() for _ in range(1)] + xs[1:]
    assert XorShift64(1).next_u64() == 0x40822041 and XorShift64(0).state == 0x9E3779B97F4A7C15


def run_late(sched, next_token, max_steps=10_000):
    """Drives the scheduler as the engine does when it reads a step's ids one step late: the next step is put
    together and launched (here: its pages checked) before the ids of the one before are resolved."""
    from ferrox_amd.engine.scheduler import UNKNOWN
    inflight = []

    def settle():
        if not inflight:
            return False
        batch, ids = inflight.pop()
        sched.resolve(batch, ids)
        sched.cache.m.check_invariants()
        return True

    sched.settle = settle
    n_steps = n_fed = 0
    while True:
        batch = sched.schedule() if sched.has_work() else []
        if not batch:
            if settle():
                continue
            assert not sched.has_work()
            break
        for s in batch:
            toks = sched.step_tokens(s)
            assert sched.cache.m.length(s.request.id) == s.request.n_computed + s.n_tokens
            assert UNKNOWN not in toks[:-1]                      # only a request's newest token can be on the way
            if toks[-1] == UNKNOWN:
                assert inflight and any(x.request is s.request and x.samples for x in inflight[0][0])
                n_fed += 1
        # the ids are what the model would give: a function of the request and of how much it has generated
        ids = {s.request.id: next_token(s.request) for s in batch if s.samples}
        settle()
        sched.commit_launched(batch)
        inflight.append((batch, ids))
        sched.cache.m.check_invariants()
        n_steps += 1
        assert n_steps < max_steps
    return n_fed


@pytest.mark.parametrize("seed", range(12))
def test_reading_the_ids_one_step_late_changes_nothing_that_is_generated(seed):
    import random
    rnd = random.Random(seed)
    n_req = rnd.randint(2, 7)
    spec = [(rnd.randint(1, 30), rnd.randint(1, 25)) for _ in range(n_req)]
    pages, budget, chunk = rnd.randint(10, 24), rnd.randint(4, 40), rnd.randint(2, 16)
    eos = 7

    def nxt(req):          # the position decides: the same token whenever and with whomever it is computed
        return (req.id * 131 + (len(req.prompt) + len(req.generated)) * 17) % 11

    outcomes = []
    for late in (False, True):
        sched = Scheduler(Cache(pages, block_size=4), max_tokens_per_step=budget, prefill_chunk=chunk, context_limit=48)
        for i, (n_prompt, n_new) in enumerate(spec):
            sched.add(Request(i, [((i + j) % 5) for j in range(n_prompt)], n_new, eos_token_id=eos, ignore_eos=(i % 3 == 2)))
        fed = run_late(sched, nxt) if late else run(sched, nxt)
        assert sched.cache.m.n_free_pages() == pages and len(sched.finished) == n_req
        assert all(t >= 0 for r in sched.finished for t in r.generated)
        outcomes.append({r.id: (r.generated, r.finish_reason) for r in sched.finished})
    assert fed > 0
    # a request that ends because the cache is full ends where the pages ran out, which may differ by the one
    # step that a request that has stopped already still holds its pages; everything else is the same
    for rid, (gen, reason) in outcomes[0].items():
        gen_late, reason_late = outcomes[1][rid]
        if "cache_full" in (reason, reason_late):
            n = min(len(gen), len(gen_late))
            assert gen[:n] == gen_late[:n]
        else:
            assert (gen, reason) == (gen_late, reason_late)
