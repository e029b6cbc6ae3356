"""Book-keeping of the cache: pages, block tables, state slots.  Host side only;
the device memory the ids point into is owned by `CacheStorage`.

Layers with the same need share a *group*: one pool of page ids and one block
table per request (a page id indexes a slab of every layer of the group).  A
group is either "all keys" (window None) or "the last W keys".  The reference
keeps one identical store per layer and never evicts (ferrox-core/src/cache.rs:331-488,
ferrox-models/src/decoder.rs:2217-2223); here a windowed group gives a page back as
soon as every position in it is older than the window of any later query.

Rules kept (and checked by `check_invariants`):
  * a page is in exactly one place: the free list or one block table;
  * `extend` either gets every page it needs in every group or changes nothing
    (ferrox-core/src/cache.rs:676-739: a failed push leaves the state unchanged);
  * `release` may be called twice (cache.rs:131-139).
Freed pages go to the top of a LIFO list and are handed out again first.
"""
from __future__ import annotations

from dataclasses import dataclass, field


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages < 0:
            raise ValueError("num_pages must be >= 0")
        self.num_pages = num_pages
        self._free = list(range(num_pages - 1, -1, -1))      # pop() hands out 0, 1, 2, ... at first
        self._is_free = [True] * num_pages

    @property
    def n_free(self) -> int:
        return len(self._free)

    def alloc(self, n: int):
        """n page ids, or None (and no change) if fewer are free."""
        if n > len(self._free):
            return None
        out = [self._free.pop() for _ in range(n)]
        for p in out:
            self._is_free[p] = False
        return out

    def free(self, pages) -> None:
        for p in pages:
            if not 0 <= p < self.num_pages:
                raise ValueError(f"page {p} does not belong to this pool")
            if self._is_free[p]:
                raise ValueError(f"page {p} freed twice")
            self._is_free[p] = True
            self._free.append(p)


class StateSlots:
    """Slots for per-request state of fixed size (sampler state, a recurrent mixer's state)."""

    def __init__(self, n_slots: int):
        self.n_slots = n_slots
        self._free = list(range(n_slots - 1, -1, -1))
        self._used: set[int] = set()

    @property
    def n_free(self) -> int:
        return len(self._free)

    def alloc(self):
        if not self._free:
            return None
        s = self._free.pop()
        self._used.add(s)
        return s

    def free(self, slot: int) -> None:
        if slot not in self._used:
            raise ValueError(f"slot {slot} is not in use")
        self._used.remove(slot)
        self._free.append(slot)


@dataclass
class Group:
    key: object
    window: int | None
    pool: PagePool
    tables: dict = field(default_factory=dict)     # request -> list of page ids, -1 where given back


@dataclass
class Sequence:
    slot: int
    length: int = 0


class CacheManager:
    def __init__(self, groups: dict, num_pages, block_size: int, n_slots: int):
        """`groups`: key -> window (None = all keys).  `num_pages`: an int for every group, or key -> int."""
        if block_size < 1:
            raise ValueError("block_size must be >= 1")
        self.block_size = block_size
        self.groups: dict = {}
        for key, window in groups.items():
            n = num_pages[key] if isinstance(num_pages, dict) else num_pages
            self.groups[key] = Group(key, window, PagePool(n))
        self.slots = StateSlots(n_slots)
        self.seqs: dict = {}

    # ---- requests --------------------------------------------------------
    def admit(self, req) -> int | None:
        """A state slot and empty block tables; None if no slot is free."""
        if req in self.seqs:
            raise ValueError(f"request {req!r} is already admitted")
        slot = self.slots.alloc()
        if slot is None:
            return None
        self.seqs[req] = Sequence(slot)
        for g in self.groups.values():
            g.tables[req] = []
        return slot

    def __contains__(self, req) -> bool:
        return req in self.seqs

    def _seq(self, req) -> Sequence:
        seq = self.seqs.get(req)
        if seq is None:
            raise ValueError(f"request {req!r} is not admitted")
        return seq

    def length(self, req) -> int:
        return self._seq(req).length

    def slot(self, req) -> int:
        return self._seq(req).slot

    def table(self, req, key) -> list:
        return self.groups[key].tables[req]

    def blocks_for(self, length: int) -> int:
        return -(-length // self.block_size)

    def pages_needed(self, req, new_len: int) -> dict:
        """key -> number of pages `extend(req, new_len)` would take."""
        return {k: max(0, self.blocks_for(new_len) - len(g.tables[req])) for k, g in self.groups.items()}

    def can_extend(self, req, new_len: int) -> bool:
        need = self.pages_needed(req, new_len)
        return all(self.groups[k].pool.n_free >= n for k, n in need.items())

    def extend(self, req, new_len: int) -> bool:
        """Pages for positions [length, new_len) in every group, all or nothing; sets the length."""
        seq = self._seq(req)
        if new_len < seq.length:
            raise ValueError("a sequence cannot shrink")
        need = self.pages_needed(req, new_len)
        if any(self.groups[k].pool.n_free < n for k, n in need.items()):
            return False
        for k, n in need.items():
            g = self.groups[k]
            g.tables[req].extend(g.pool.alloc(n))
        seq.length = new_len
        return True

    def trim(self, req) -> int:
        """Give back pages that a window has passed: every query from now on stands at
        position >= length and sees keys t with position - t < W, so t >= length - W + 1.
        Returns the number of pages freed."""
        seq = self._seq(req)
        freed = 0
        for g in self.groups.values():
            if g.window is None:
                continue
            first_needed = seq.length - g.window + 1
            if first_needed <= 0:
                continue
            table = g.tables[req]
            for b in range(min(first_needed // self.block_size, len(table))):
                if table[b] >= 0:
                    g.pool.free([table[b]])
                    table[b] = -1
                    freed += 1
        return freed

    def release(self, req) -> None:
        """Everything the request holds goes back; a second call does nothing."""
        seq = self.seqs.pop(req, None)
        if seq is None:
            return
        for g in self.groups.values():
            g.pool.free([p for p in g.tables.pop(req) if p >= 0])
        self.slots.free(seq.slot)

    # ---- accounting --------------------------------------------------------
    def n_free_pages(self, key=None) -> int:
        if key is not None:
            return self.groups[key].pool.n_free
        return min(g.pool.n_free for g in self.groups.values()) if self.groups else 0

    def check_invariants(self) -> None:
        for g in self.groups.values():
            held = [p for t in g.tables.values() for p in t if p >= 0]
            if len(held) != len(set(held)):
                raise AssertionError(f"group {g.key!r}: a page is held twice")
            free = list(g.pool._free)
            if len(free) != len(set(free)):
                raise AssertionError(f"group {g.key!r}: a page is in the free list twice")
            if set(free) & set(held):
                raise AssertionError(f"group {g.key!r}: a page is both free and held")
            if len(free) + len(held) != g.pool.num_pages:
                raise AssertionError(f"group {g.key!r}: {g.pool.num_pages - len(free) - len(held)} pages lost")
            if set(g.tables) != set(self.seqs):
                raise AssertionError(f"group {g.key!r}: tables and sequences differ")
            for req, t in g.tables.items():
                if len(t) < self.blocks_for(self.seqs[req].length):
                    raise AssertionError(f"group {g.key!r}: request {req!r} has too few blocks")
        slots = [s.slot for s in self.seqs.values()]
        if len(slots) != len(set(slots)):
            raise AssertionError("a state slot is held twice")
        if len(slots) + self.slots.n_free != self.slots.n_slots:
            raise AssertionError("state slots lost")
