"""Book-keeping of the cache: pages, block tables, state slots.  Host side only;
the device memory the ids point into is owned by `CacheStorage`.

The book-keeping itself is native code (`csrc/host_runtime.cpp`, loaded through
ctypes); this module is its Python face: it maps request names to handles and
group keys to indexes, and turns error codes into exceptions.

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

import ctypes

import numpy as np

from ..csrc.build import load_library

_I32P = ctypes.POINTER(ctypes.c_int)
_I64P = ctypes.POINTER(ctypes.c_int64)
_lib = None


def _native():
    global _lib
    if _lib is None:
        lib = load_library("host_runtime")
        lib.fxc_create.restype = ctypes.c_void_p
        lib.fxc_create.argtypes = [ctypes.c_int, _I32P, _I32P, ctypes.c_int, ctypes.c_int]
        lib.fxc_destroy.argtypes = [ctypes.c_void_p]
        lib.fxc_destroy.restype = None
        lib.fxc_last_error.restype = ctypes.c_char_p
        lib.fxc_last_error.argtypes = [ctypes.c_void_p]
        for name, extra in (("admit", []), ("contains", []), ("length", []), ("slot", []), ("trim", []),
                            ("pages_needed", [ctypes.c_int, ctypes.c_int]), ("extend", [ctypes.c_int, ctypes.c_int]),
                            ("table", [ctypes.c_int, _I32P, ctypes.c_int])):
            fn = getattr(lib, "fxc_" + name)
            fn.restype = ctypes.c_int
            fn.argtypes = [ctypes.c_void_p, ctypes.c_int64] + extra
        lib.fxc_release.restype = None
        lib.fxc_release.argtypes = [ctypes.c_void_p, ctypes.c_int64]
        for name, extra in (("n_free_pages", [ctypes.c_int]), ("num_pages", [ctypes.c_int]), ("n_free_slots", []),
                            ("n_requests", []), ("check", []), ("pool_take", [ctypes.c_int, ctypes.c_int, _I32P]),
                            ("pool_give", [ctypes.c_int, ctypes.c_int]), ("slot_take", []), ("slot_give", [ctypes.c_int])):
            fn = getattr(lib, "fxc_" + name)
            fn.restype = ctypes.c_int
            fn.argtypes = [ctypes.c_void_p] + extra
        lib.fxc_pack_step.restype = ctypes.c_long
        lib.fxc_pack_step.argtypes = [ctypes.c_void_p, ctypes.c_int, _I64P, _I32P, _I32P, _I32P, _I32P, ctypes.c_int,
                                      ctypes.c_int, ctypes.c_void_p, ctypes.c_long, _I32P, _I32P, _I32P]
        lib.fxc_pack_decode.restype = ctypes.c_long
        lib.fxc_pack_decode.argtypes = [ctypes.c_void_p, ctypes.c_int, _I64P, _I32P, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                        _I32P, ctypes.c_int, ctypes.c_void_p, ctypes.c_long, _I32P]
        _lib = lib
    return _lib


class _Core:
    """Owns one native manager."""

    def __init__(self, windows: list, num_pages: list, block_size: int, n_slots: int):
        for n in num_pages:
            if n < 0:
                raise ValueError("num_pages must be >= 0")
        if block_size < 1:
            raise ValueError("block_size must be >= 1")
        self.lib = _native()
        n = len(windows)
        w = (ctypes.c_int * max(n, 1))(*[-1 if x is None else int(x) for x in windows])
        p = (ctypes.c_int * max(n, 1))(*[int(x) for x in num_pages])
        self.h = self.lib.fxc_create(n, w, p, block_size, n_slots)
        if not self.h:
            raise ValueError("the cache manager refused its sizes")

    def __del__(self):
        h, self.h = getattr(self, "h", None), None
        if h:
            self.lib.fxc_destroy(h)

    def error(self) -> str:
        return self.lib.fxc_last_error(self.h).decode()


class PagePool:
    """One pool of page ids on its own."""

    def __init__(self, num_pages: int):
        self._core = _Core([None], [num_pages], 1, 0)
        self.num_pages = num_pages

    @property
    def n_free(self) -> int:
        return self._core.lib.fxc_n_free_pages(self._core.h, 0)

    def alloc(self, n: int):
        """n page ids, or None (and no change) if fewer are free."""
        out = (ctypes.c_int * max(n, 1))()
        if not self._core.lib.fxc_pool_take(self._core.h, 0, n, out):
            return None
        return list(out[:n])

    def free(self, pages) -> None:
        for p in pages:
            if not self._core.lib.fxc_pool_give(self._core.h, 0, int(p)):
                raise ValueError(f"page {p} does not belong to this pool or is freed twice")


class StateSlots:
    """Slots for per-request state of fixed size (sampler state, a recurrent mixer's state)."""

    def __init__(self, n_slots: int):
        self._core = _Core([], [], 1, n_slots)
        self.n_slots = n_slots

    @property
    def n_free(self) -> int:
        return self._core.lib.fxc_n_free_slots(self._core.h)

    def alloc(self):
        s = self._core.lib.fxc_slot_take(self._core.h)
        return None if s < 0 else s

    def free(self, slot: int) -> None:
        if not self._core.lib.fxc_slot_give(self._core.h, int(slot)):
            raise ValueError(f"slot {slot} is not in use")


class _PoolView:
    def __init__(self, mgr, index):
        self._m, self._g = mgr, index

    @property
    def n_free(self) -> int:
        return self._m._lib.fxc_n_free_pages(self._m._h, self._g)

    @property
    def num_pages(self) -> int:
        return self._m._lib.fxc_num_pages(self._m._h, self._g)


class _TablesView:
    def __init__(self, mgr, key):
        self._m, self._key = mgr, key

    def __getitem__(self, req) -> list:
        return self._m.table(req, self._key)


class Group:
    """What one group shows: its key, its window, its pool's counts and the block tables."""

    def __init__(self, mgr, key, window, index):
        self.key, self.window, self.index = key, window, index
        self.pool = _PoolView(mgr, index)
        self.tables = _TablesView(mgr, key)


class _SlotsView:
    def __init__(self, mgr, n_slots):
        self._m, self.n_slots = mgr, n_slots

    @property
    def n_free(self) -> int:
        return self._m._lib.fxc_n_free_slots(self._m._h)


class PackedStep:
    """A step's batch as the native packer laid it out in a host int32 buffer:
    tokens[T] | positions[T] | token_seq[T] | slots[n] | rows[R] | tables[groups][n][max_blocks]."""
    __slots__ = ("total", "n_tokens", "n_rows", "max_blocks", "starts", "lens")

    def __init__(self, total, n_tokens, n_rows, max_blocks, starts, lens):
        self.total, self.n_tokens, self.n_rows, self.max_blocks = total, n_tokens, n_rows, max_blocks
        self.starts, self.lens = starts, lens


class CacheManager:
    def __init__(self, groups: dict, num_pages, block_size: int, n_slots: int):
        """`groups`: key -> window (None = all keys).  `num_pages`: an int for every group, or key -> int."""
        keys = list(groups)
        pages = [num_pages[k] if isinstance(num_pages, dict) else num_pages for k in keys]
        self._core = _Core([groups[k] for k in keys], pages, block_size, n_slots)
        self._lib, self._h = self._core.lib, self._core.h
        self.block_size = block_size
        self.groups = {k: Group(self, k, groups[k], i) for i, k in enumerate(keys)}
        self.slots = _SlotsView(self, n_slots)
        self._handles: dict = {}        # request name -> handle
        self._next = 0
        self._decode_arrays = None      # what pack_decode keeps between steps

    # ---- requests --------------------------------------------------------
    def _handle(self, req) -> int:
        h = self._handles.get(req)
        if h is None:
            raise ValueError(f"request {req!r} is not admitted")
        return h

    def _checked(self, code: int) -> int:
        if code == -2:
            raise ValueError(self._core.error())
        return code

    def admit(self, req) -> int | None:
        """A state slot and empty block tables; None if no slot is free."""
        if req in self._handles:
            raise ValueError(f"request {req!r} is already admitted")
        slot = self._checked(self._lib.fxc_admit(self._h, self._next))
        if slot < 0:
            return None
        self._handles[req] = self._next
        self._next += 1
        return slot

    def __contains__(self, req) -> bool:
        return req in self._handles

    @property
    def seqs(self) -> dict:
        """request -> length, for inspection"""
        return {r: self.length(r) for r in self._handles}

    def length(self, req) -> int:
        return self._checked(self._lib.fxc_length(self._h, self._handle(req)))

    def slot(self, req) -> int:
        return self._checked(self._lib.fxc_slot(self._h, self._handle(req)))

    def table(self, req, key) -> list:
        h, g = self._handle(req), self.groups[key].index
        n = self._checked(self._lib.fxc_table(self._h, h, g, None, 0))
        out = (ctypes.c_int * max(n, 1))()
        self._lib.fxc_table(self._h, h, g, out, n)
        return list(out[:n])

    def blocks_for(self, length: int) -> int:
        return -(-length // self.block_size)

    def pages_needed(self, req, new_len: int) -> dict:
        """key -> number of pages `extend(req, new_len)` would take."""
        h = self._handle(req)
        return {k: self._checked(self._lib.fxc_pages_needed(self._h, h, new_len, g.index))
                for k, g in self.groups.items()}

    def can_extend(self, req, new_len: int) -> bool:
        return self._checked(self._lib.fxc_extend(self._h, self._handle(req), new_len, 1)) == 1

    def extend(self, req, new_len: int) -> bool:
        """Pages for positions [length, new_len) in every group, all or nothing; sets the length."""
        return self._checked(self._lib.fxc_extend(self._h, self._handle(req), new_len, 0)) == 1

    def trim(self, req) -> int:
        """Give back pages that a window has passed: every query from now on stands at
        position >= length and sees keys t with position - t < W, so t >= length - W + 1.
        Returns the number of pages freed."""
        return self._checked(self._lib.fxc_trim(self._h, self._handle(req)))

    def release(self, req) -> None:
        """Everything the request holds goes back; a second call does nothing."""
        h = self._handles.pop(req, None)
        if h is not None:
            self._decode_arrays = None
            self._lib.fxc_release(self._h, h)

    # ---- the step's batch ----------------------------------------------------
    def pack_step(self, reqs: list, token_lists: list, wants: list, vocab: int, out_ptr: int, capacity: int,
                  force_blocks: int = 0) -> PackedStep:
        """Lay the batch out in the host buffer at `out_ptr` (room for `capacity` int32).
        Checks every id and place; raises ValueError naming the request at fault."""
        n = len(reqs)
        handles = np.empty(n, dtype=np.int64)
        for i, r in enumerate(reqs):
            h = self._handles.get(r)
            if h is None:
                raise ValueError(f"request {r!r} was not admitted")
            handles[i] = h
        n_tok = np.fromiter((len(t) for t in token_lists), dtype=np.int32, count=n)
        try:
            tokens = np.concatenate([np.asarray(t, dtype=np.int64).reshape(-1) for t in token_lists]) if n else \
                np.empty(0, dtype=np.int64)
            flat_want = np.concatenate([np.asarray(w, dtype=np.int64).reshape(-1) for w in wants]) if n else \
                np.empty(0, dtype=np.int64)
        except (OverflowError, TypeError, ValueError) as e:
            raise ValueError(f"token ids and wanted places must be integers: {e}") from None
        if tokens.size and (tokens.min() < 0 or tokens.max() >= vocab):
            bad = int(tokens[(tokens < 0) | (tokens >= vocab)][0])
            raise ValueError(f"token id {bad} is outside the vocabulary of {vocab}")     # ferrox-cli/src/run.rs:598-601
        if flat_want.size and (flat_want.min() < -(2 ** 31) or flat_want.max() >= 2 ** 31):
            raise ValueError("a wanted place is outside its request's tokens")
        tokens, flat_want = tokens.astype(np.int32), flat_want.astype(np.int32)
        want_start = np.zeros(n + 1, dtype=np.int32)
        np.cumsum([len(w) for w in wants], out=want_start[1:])
        sizes = np.zeros(3, dtype=np.int32)
        starts, lens = np.zeros(max(n, 1), dtype=np.int32), np.zeros(max(n, 1), dtype=np.int32)
        ip = lambda a: a.ctypes.data_as(_I32P)
        total = self._lib.fxc_pack_step(self._h, n, handles.ctypes.data_as(_I64P), ip(n_tok), ip(tokens), ip(want_start),
                                        ip(flat_want), vocab, force_blocks, out_ptr, capacity, ip(sizes), ip(starts),
                                        ip(lens))
        if total < 0:
            msg = self._core.error()
            by_handle = {h: r for r, h in self._handles.items()}
            for h, r in by_handle.items():              # name the request as the caller knows it
                msg = msg.replace(f"request {h} ", f"request {r!r} ").replace(f"request {h}:", f"request {r!r}:")
            raise ValueError(msg)
        return PackedStep(int(total), int(sizes[0]), int(sizes[1]), int(sizes[2]), starts[:n].tolist(), lens[:n].tolist())

    def pack_decode(self, reqs: list, tokens: list, vocab: int, out_ptr: int, capacity: int, force_blocks: int,
                    pad_to: int | None = None, pad_pages: list | None = None, pad_slot: int = 0) -> None:
        """The common step in which every request brings one token and wants its logits, laid out for
        `pad_to` >= len(reqs) sequences: the rows past the requests are stand-ins that write to the page
        `pad_pages[group]` and the state slot `pad_slot`, which no request owns.  The arrays that do not
        change from step to step are kept from the last call."""
        n = len(reqs)
        key = tuple(reqs)
        kept = self._decode_arrays
        if kept is None or kept[0] != key:
            handles = np.empty(n, dtype=np.int64)
            for i, r in enumerate(reqs):
                h = self._handles.get(r)
                if h is None:
                    raise ValueError(f"request {r!r} was not admitted")
                handles[i] = h
            kept = self._decode_arrays = (key, handles, np.zeros(n, dtype=np.int32))
        _, handles, lens = kept
        try:
            toks = np.asarray(tokens, dtype=np.int32).reshape(-1)
        except (OverflowError, TypeError, ValueError) as e:
            raise ValueError(f"token ids must be integers: {e}") from None
        if toks.size != n:
            raise ValueError("one token per request")
        pads = np.asarray(pad_pages if pad_pages is not None else [0] * len(self.groups), dtype=np.int32)
        if pads.size != len(self.groups):
            raise ValueError("one stand-in page per group")
        ip = lambda a: a.ctypes.data_as(_I32P)
        total = self._lib.fxc_pack_decode(self._h, n, handles.ctypes.data_as(_I64P), ip(toks), vocab, force_blocks,
                                          n if pad_to is None else int(pad_to), ip(pads), int(pad_slot), out_ptr, capacity,
                                          ip(lens))
        if total < 0:
            self._decode_arrays = None
            raise ValueError(self._core.error())

    def step_words(self, n_tokens: int, n_seqs: int, n_rows: int, max_blocks: int) -> int:
        return 3 * n_tokens + n_seqs + n_rows + len(self.groups) * n_seqs * max_blocks

    # ---- accounting --------------------------------------------------------
    def n_free_pages(self, key=None) -> int:
        if key is not None:
            return self.groups[key].pool.n_free
        return min(g.pool.n_free for g in self.groups.values()) if self.groups else 0

    def check_invariants(self) -> None:
        if self._lib.fxc_check(self._h) != 0:
            raise AssertionError(self._core.error())
        if self._lib.fxc_n_requests(self._h) != len(self._handles):
            raise AssertionError("requests known to the manager and to its core differ")
