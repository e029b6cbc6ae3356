"""A model built from a `ModelSpec`: embedding, blocks, the order they run in,
final norm and head.  It owns the weights; the cache belongs to the runner."""
from __future__ import annotations

import torch

from .. import debug
from ..parts.base import (BLOCKS, EMBEDDINGS, HEADS, NORMS, LayerCache, ModelSpec, StepContext, walk_params,
                          walk_parts)
from ..weights.loader import check_names, upload


class Fetcher:
    """What a part's `load` receives: `fetch(local name)` for its own tensors, `fetch.shared(full name)` for one
    that another part owns and this part has announced in `borrows()`."""

    def __init__(self, get, prefix: str, shared: dict):
        self._get, self._prefix, self._shared = get, prefix, shared

    def __call__(self, local: str) -> torch.Tensor:
        return self._get(self._prefix + local)

    def shared(self, name: str) -> torch.Tensor:
        if name not in self._shared:
            raise KeyError(f"part '{self._prefix}' asks for '{name}' without having announced it in borrows()")
        return self._get(name)


class Model:
    def __init__(self, spec: ModelSpec):
        self.spec = spec
        self.embedding = EMBEDDINGS.build(spec.embedding)
        self.blocks = []
        for ls in spec.layers:
            cls = BLOCKS.get(ls.block)
            missing = set(cls.slots) - set(ls.parts)
            if missing:
                raise ValueError(f"layer {ls.prefix!r}: block '{ls.block}' needs parts {sorted(missing)}")
            parts = {slot: reg.build(ls.parts[slot]) for slot, reg in cls.slots.items()}
            self.blocks.append(cls(parts, {slot: ls.parts[slot].prefix for slot in cls.slots}))
        self.final_norm = NORMS.build(spec.final_norm)
        self.head = HEADS.build(spec.head)
        self.schedule = list(spec.schedule)
        for i, e in enumerate(self.schedule):
            if not 0 <= e.layer < len(self.blocks):
                raise ValueError(f"schedule entry {i} names layer {e.layer}; the model has {len(self.blocks)}")
            if e.cache is not None:
                if not 0 <= e.cache < i or self.schedule[e.cache].cache is not None:
                    raise ValueError(f"schedule entry {i} reads the cache of entry {e.cache}, which must be an "
                                     f"earlier entry with a cache of its own")
                a, b = self.blocks[e.layer].mixer, self.blocks[self.schedule[e.cache].layer].mixer
                if a.cache_group() != b.cache_group() or a.page_shapes(16) != b.page_shapes(16):
                    raise ValueError(f"schedule entry {i} cannot read the cache of entry {e.cache}: "
                                     f"their mixers keep different pages")
        self.act_dtype = None
        self.device = None

    # ---- parameters ------------------------------------------------------
    def _roots(self):
        yield self.spec.embedding.prefix, self.embedding
        for ls, block in zip(self.spec.layers, self.blocks):
            yield ls.prefix, block
        yield self.spec.final_norm.prefix, self.final_norm
        yield self.spec.head.prefix, self.head

    def named_params(self) -> dict:
        out = {}
        for prefix, root in self._roots():
            for name, spec, _, _ in walk_params(root, prefix):
                if name in out:
                    raise ValueError(f"two parts claim the tensor '{name}'")
                out[name] = spec
        return out

    def kernel_libraries(self) -> list:
        libs = []
        for prefix, root in self._roots():
            for _, part in walk_parts(root, prefix):
                for lib in part.kernel_libraries:
                    if lib not in libs:
                        libs.append(lib)
        return libs

    def load(self, source, act_dtype: torch.dtype, device, where: str = "") -> None:
        """Check every name and shape first (one error for all), then upload part by part."""
        if hasattr(source, "expect"):
            source.expect(self.named_params())
        check_names(self.named_params(), source, where)
        device = torch.device(device)
        owned = self.named_params()
        shared: dict = {}              # full name -> the one tensor that its owner and its borrowers get
        for prefix, root in self._roots():
            for pfx, part in walk_parts(root, prefix):
                for name in part.borrows():
                    if name not in owned:
                        raise ValueError(f"part '{pfx}' ({type(part).__name__}) reads the tensor '{name}', "
                                         f"which no part of the model declares")
                    shared[name] = None

        def get(name: str) -> torch.Tensor:
            if name not in shared:
                return upload(source, name, act_dtype, device)
            if shared[name] is None:
                shared[name] = upload(source, name, act_dtype, device)
            return shared[name]

        for prefix, root in self._roots():
            for pfx, part in walk_parts(root, prefix):
                part.load(Fetcher(get, pfx, shared))
        self.act_dtype, self.device = act_dtype, device

    # ---- cache needs -----------------------------------------------------
    def cache_groups(self) -> dict:
        """group key -> window, over the mixers that keep pages."""
        groups = {}
        for e in self.schedule:
            m = self.blocks[e.layer].mixer
            if m.page_shapes(16):
                key, window = m.cache_group()
                if groups.setdefault(key, window) != window:
                    raise ValueError(f"two mixers name the cache group {key!r} with windows {groups[key]} and {window}")
        return groups

    # ---- forward ---------------------------------------------------------
    def forward(self, ctx: StepContext, caches: list):
        debug.region("embed")
        h = self.embedding.forward(ctx.token_ids)
        # blocks that chain their norms: the block before may already have applied this block's first norm
        # to the rows it finished (in the kernel that finished them)
        normed = None
        for i, e in enumerate(self.schedule):
            block = self.blocks[e.layer]
            if block.chains_norms:
                nxt = self.blocks[self.schedule[i + 1].layer] if i + 1 < len(self.schedule) else None
                then = (nxt.first_norm, nxt.takes_scale_later(ctx.act_dtype)) \
                    if nxt is not None and nxt.chains_norms else None
                normed = block.forward(h, ctx, caches[i], normed=normed, then=then)
            else:
                block.forward(h, ctx, caches[i])
                normed = None
        if ctx.logit_rows is None or ctx.logit_rows.numel() == 0:
            return None
        debug.region("final norm")
        x = self.final_norm.forward(h, ctx, rows=ctx.logit_rows)
        debug.region("head")
        return self.head.forward(x)
