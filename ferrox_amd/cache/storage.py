"""Device memory behind the cache manager's page ids and slot ids.

Each schedule entry with a cache of its own gets, for every page tensor its
mixer names, a slab [num_pages + 1, *page_shape], and for every state tensor a slab
[n_slots + 1, *state_shape].  An entry that reads another entry's cache sees that
entry's page slabs, read-only.  The one page and the one slot past the manager's
own belong to no request: the stand-in rows that fill a recorded decode step up
to its fixed number of sequences write there (`pad_page`, `pad_slot`).
"""
from __future__ import annotations

import torch

from ..parts.base import LayerCache


class CacheStorage:
    def __init__(self, model, manager, dtype: torch.dtype, device):
        self.caches: list[LayerCache] = []
        self.bytes = 0
        self.pad_pages = [g.pool.num_pages for g in manager.groups.values()]     # per group, in the manager's order
        self.pad_slot = manager.slots.n_slots
        bs = manager.block_size
        for i, e in enumerate(model.schedule):
            mixer = model.blocks[e.layer].mixer
            shapes = mixer.page_shapes(bs)
            key = mixer.cache_group()[0] if shapes else None
            state = {}
            for name, (shape, sdtype) in mixer.state_shapes().items():
                state[name] = torch.zeros((manager.slots.n_slots + 1, *shape), dtype=sdtype or dtype, device=device)
                self.bytes += state[name].numel() * state[name].element_size()
            if e.cache is not None:
                owner = self.caches[e.cache]
                self.caches.append(LayerCache(owner.pages, state, key, bs, writes=False))
                continue
            pages = {}
            if shapes:
                n = manager.groups[key].pool.num_pages
                for name, shape in shapes.items():
                    pages[name] = torch.zeros((n + 1, *shape), dtype=dtype, device=device)
                    self.bytes += pages[name].numel() * pages[name].element_size()
            self.caches.append(LayerCache(pages, state, key, bs, writes=True))

    def clear_slot(self, slot: int) -> None:
        """State of a newly admitted request starts at zero."""
        for c in self.caches:
            for t in c.state.values():
                t[slot].zero_()
