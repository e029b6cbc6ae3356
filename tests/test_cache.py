"""The cache manager: no page lost, held twice or freed twice, under random orders of requests."""
import random

import pytest

from ferrox_amd.cache import CacheManager, PagePool, StateSlots

FULL, WIN = ("full",), ("window", 16)


def test_pool_hands_out_and_takes_back():
    pool = PagePool(4)
    a = pool.alloc(3)
    assert a == [0, 1, 2] and pool.n_free == 1
    assert pool.alloc(2) is None and pool.n_free == 1              # all or nothing, nothing changed
    pool.free([1])
    assert pool.alloc(1) == [1]                                    # the page just freed is used again first
    with pytest.raises(ValueError):
        pool.free([3])                                             # never handed out
    pool.free([0])
    with pytest.raises(ValueError):
        pool.free([0])                                             # freed twice
    with pytest.raises(ValueError):
        pool.free([9])


def test_slots():
    s = StateSlots(2)
    a, b = s.alloc(), s.alloc()
    assert {a, b} == {0, 1} and s.alloc() is None
    s.free(a)
    assert s.alloc() == a
    with pytest.raises(ValueError):
        s.free(5)


def test_extend_is_all_or_nothing_across_groups():
    m = CacheManager({FULL: None, WIN: 16}, {FULL: 4, WIN: 2}, block_size=8, n_slots=2)
    assert m.admit("a") == 0
    assert m.extend("a", 16) and m.length("a") == 16               # 2 pages in both groups
    before = (m.n_free_pages(FULL), m.n_free_pages(WIN), list(m.table("a", FULL)))
    assert not m.can_extend("a", 17) and not m.extend("a", 17)     # the windowed pool is empty
    assert (m.n_free_pages(FULL), m.n_free_pages(WIN), list(m.table("a", FULL))) == before and m.length("a") == 16
    m.check_invariants()
    m.release("a")
    m.release("a")                                                 # twice is fine (cache.rs:131-139)
    assert m.n_free_pages(FULL) == 4 and m.n_free_pages(WIN) == 2 and m.slots.n_free == 2
    with pytest.raises(ValueError):
        m.extend("a", 4)


def test_window_gives_pages_back_when_they_are_passed():
    m = CacheManager({FULL: None, WIN: 16}, 16, block_size=8, n_slots=1)
    m.admit("r")
    m.extend("r", 40)
    assert m.trim("r") == 3                   # next query stands at 40 and sees 25..40: blocks 0, 1, 2 are passed
    assert m.table("r", WIN)[:3] == [-1, -1, -1] and all(p >= 0 for p in m.table("r", WIN)[3:])
    assert all(p >= 0 for p in m.table("r", FULL))                 # the full group keeps everything
    assert m.trim("r") == 0
    m.extend("r", 41)
    assert m.trim("r") == 0                   # first key still needed is 26, in block 3
    m.extend("r", 47)
    assert m.trim("r") == 1                   # 47 - 16 + 1 = 32: block 3 is passed
    m.check_invariants()
    m.release("r")
    assert m.n_free_pages(WIN) == 16 and m.n_free_pages(FULL) == 16


def test_pages_of_a_finished_request_are_used_again():
    m = CacheManager({FULL: None}, 3, block_size=4, n_slots=2)
    m.admit("a")
    m.extend("a", 12)
    pages = list(m.table("a", FULL))
    m.admit("b")
    assert not m.extend("b", 1)
    m.release("a")
    assert m.extend("b", 12) and sorted(m.table("b", FULL)) == sorted(pages)


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_the_invariants(seed):
    rng = random.Random(seed)
    m = CacheManager({FULL: None, WIN: 16, ("window", 40): 40}, {FULL: 40, WIN: 12, ("window", 40): 20},
                     block_size=rng.choice([4, 8, 16]), n_slots=4)
    live, next_id = {}, 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and len(live) < 5:
            rid = f"r{next_id}"
            next_id += 1
            if m.admit(rid) is not None:
                live[rid] = 0
            else:
                assert len(live) == 4
        elif op < 0.8 and live:
            rid = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 5, 13, 30])
            had = {k: m.n_free_pages(k) for k in m.groups}
            if m.extend(rid, live[rid] + n):
                live[rid] += n
                m.trim(rid)
            else:
                assert {k: m.n_free_pages(k) for k in m.groups} == had
        elif live:
            rid = rng.choice(list(live))
            m.release(rid)
            del live[rid]
        m.check_invariants()
        for rid, n in live.items():
            assert m.length(rid) == n
            # every position a later query can see has a page in every group
            for g in m.groups.values():
                first = 0 if g.window is None else max(0, n - g.window + 1)
                assert all(g.tables[rid][b] >= 0 for b in range(first // m.block_size, m.blocks_for(n)))
    for rid in list(live):
        m.release(rid)
    m.check_invariants()
    assert all(g.pool.n_free == g.pool.num_pages for g in m.groups.values()) and m.slots.n_free == 4


def _pack(m, reqs, toks, wants, vocab=100, force=0, cap=4096):
    import numpy as np
    buf = np.full(cap, -7, dtype=np.int32)
    p = m.pack_step(reqs, toks, wants, vocab, buf.ctypes.data, cap, force_blocks=force)
    return p, buf


def test_pack_step_layout():
    m = CacheManager({FULL: None, WIN: 16}, 16, block_size=8, n_slots=4)
    for r, n in (("a", 21), ("b", 40)):
        m.admit(r)
        m.extend(r, n)
    m.trim("b")                                                    # b's first windowed blocks are given back
    p, buf = _pack(m, ["b", "a"], [[7], [1, 2, 3]], [[0], [0, 2]])
    T, n, R, mb = 4, 2, 3, 5
    assert (p.n_tokens, p.n_rows, p.max_blocks, p.total) == (T, R, mb, 3 * T + n + R + 2 * n * mb)
    assert p.starts == [39, 18] and p.lens == [40, 21]
    assert buf[:T].tolist() == [7, 1, 2, 3]
    assert buf[T:2 * T].tolist() == [39, 18, 19, 20]               # positions go on where the cache ends
    assert buf[2 * T:3 * T].tolist() == [0, 1, 1, 1]
    assert buf[3 * T:3 * T + n].tolist() == [m.slot("b"), m.slot("a")]
    assert buf[3 * T + n:3 * T + n + R].tolist() == [0, 1, 3]      # rows of the flat batch
    o = 3 * T + n + R
    full_b, full_a = m.table("b", FULL), m.table("a", FULL)
    assert buf[o:o + mb].tolist() == full_b and buf[o + mb:o + 2 * mb].tolist() == full_a + [0, 0]
    win_b = [max(x, 0) for x in m.table("b", WIN)]                 # freed entries are written as 0, never read
    assert buf[o + 2 * mb:o + 3 * mb].tolist() == win_b and m.table("b", WIN)[:3] == [-1, -1, -1]
    assert buf[p.total] == -7                                      # nothing written past the end
    p2, buf2 = _pack(m, ["b", "a"], [[7], [1, 2, 3]], [[0], [0, 2]], force=9)
    assert p2.max_blocks == 9 and buf2[o:o + 9].tolist() == full_b + [0] * 4


def test_pack_step_refuses_what_does_not_fit():
    m = CacheManager({FULL: None}, 8, block_size=8, n_slots=4)
    m.admit("a")
    m.extend("a", 3)
    for reqs, toks, wants, word in (
            (["zz"], [[1]], [[0]], "not admitted"),
            (["a"], [[]], [[]], "no tokens"),
            (["a"], [[1, 2, 3, 4]], [[]], "reserved"),
            (["a"], [[1, 100]], [[]], "vocabulary"),
            (["a"], [[1, -1]], [[]], "vocabulary"),
            (["a"], [[1, 2]], [[2]], "wanted place"),
            (["a", "a"], [[1], [2]], [[], []], "twice")):
        with pytest.raises(ValueError, match=word):
            _pack(m, reqs, toks, wants)
    with pytest.raises(ValueError, match="too small"):
        _pack(m, ["a"], [[1, 2]], [[1]], cap=4)
    with pytest.raises(ValueError, match="cannot hold"):
        m.extend("a", 20)
        _pack(m, ["a"], [[1, 2]], [[1]], force=2)
    m.check_invariants()


def test_pack_decode_writes_what_pack_step_writes():
    import numpy as np
    m = CacheManager({FULL: None, WIN: 16}, 16, block_size=8, n_slots=4)
    for r, n in (("a", 21), ("b", 40), ("c", 9)):
        m.admit(r)
        m.extend(r, n)
    for reqs, toks in ((["b", "a", "c"], [7, 1, 3]), (["b", "a", "c"], [9, 9, 2]), (["c", "b"], [5, 6])):
        want, buf = _pack(m, reqs, [[t] for t in toks], [[0]] * len(reqs), force=6)
        got = np.full(4096, -7, dtype=np.int32)
        m.pack_decode(reqs, toks, 100, got.ctypes.data, 4096, 6)
        assert (got == buf).all()
    m.release("b")                     # what was kept for (c, b) must not outlive b
    m.admit("b")
    m.extend("b", 3)
    want, buf = _pack(m, ["c", "b"], [[5], [6]], [[0], [0]], force=6)
    got = np.full(4096, -7, dtype=np.int32)
    m.pack_decode(["c", "b"], [5, 6], 100, got.ctypes.data, 4096, 6)
    assert (got == buf).all()
    with pytest.raises(ValueError, match="vocabulary"):
        m.pack_decode(["c", "b"], [5, 100], 100, got.ctypes.data, 4096, 6)
    with pytest.raises(ValueError, match="not admitted"):
        m.pack_decode(["zz"], [5], 100, got.ctypes.data, 4096, 6)


def test_pack_decode_fills_up_with_stand_in_rows():
    """a recorded step has a fixed number of sequences: the rows past the requests are a token 0 at position 0 of a
    sequence whose only block is the group's stand-in page and whose state slot is the stand-in slot"""
    import numpy as np
    m = CacheManager({FULL: None, WIN: 16}, 16, block_size=8, n_slots=4)
    for r, n in (("a", 21), ("b", 40)):
        m.admit(r)
        m.extend(r, n)
    N, mb = 5, 6
    got = np.full(4096, -7, dtype=np.int32)
    m.pack_decode(["b", "a"], [7, 3], 100, got.ctypes.data, 4096, mb, pad_to=N, pad_pages=[16, 17], pad_slot=4)
    assert got[:N].tolist() == [7, 3, 0, 0, 0]
    assert got[N:2 * N].tolist() == [39, 20, 0, 0, 0]
    assert got[2 * N:3 * N].tolist() == [0, 1, 2, 3, 4] and got[4 * N:5 * N].tolist() == [0, 1, 2, 3, 4]
    assert got[3 * N:4 * N].tolist() == [m.slot("b"), m.slot("a"), 4, 4, 4]
    o = 5 * N
    assert got[o:o + mb].tolist() == m.table("b", FULL) + [0] and got[o + mb:o + 2 * mb].tolist() == m.table("a", FULL) + [0] * 3
    assert got[o + 2 * mb:o + 5 * mb].tolist() == [16] * (3 * mb)                   # stand-ins, group FULL
    o += N * mb
    assert got[o:o + mb].tolist() == [max(x, 0) for x in m.table("b", WIN)] + [0]
    assert got[o + 2 * mb:o + 5 * mb].tolist() == [17] * (3 * mb)                   # stand-ins, group WIN
    assert got[5 * N + 2 * N * mb] == -7
    with pytest.raises(ValueError, match="cannot be laid out"):
        m.pack_decode(["b", "a"], [7, 3], 100, got.ctypes.data, 4096, mb, pad_to=1, pad_pages=[16, 17], pad_slot=4)
    m.check_invariants()
