"""What a model is put together from, and the registries the parts are found in.

A model is data: a `ModelSpec` lists an embedding, layers (each a block made of
a mixer, a feed-forward and norms, every one a `PartSpec` = kind + arguments),
the order in which the layers run (`schedule`), a final norm and a head.  The
builder looks each kind up in a registry and constructs it from its arguments;
no part knows which model it is in.  Another part becomes available by
registering a class under a new kind; nothing else changes.

Interfaces (all tensors on the GPU; `h` is the float32 residual stream [T, H],
`x` an activation [T, H] in `ctx.act_dtype`):

  Norm             forward(h, ctx, rows=None) -> x
  PositionEncoding rotary() -> a `Rotary` (dimension, theta, pairing, optional table of
                   per-pair frequency factors) when the attention kernels can apply it
                   themselves, else None and
                   apply(q, k, ctx) -> None rotates q [T, nh*hd], k [T, nkv*hd] in place
  Mixer            window (None or int), page_shapes(block_size) -> {name: shape},
                   cache_group() -> (key, window), state_shapes() -> {name: (shape, dtype)}, graph_safe,
                   forward(x, ctx, cache, residual) -> None   (adds its output into residual)
  FeedForward      forward(x, ctx, residual) -> None
  Block            forward(h, ctx, cache) -> None
  every part       param_specs() -> {local name: ParamSpec}, load(fetch), kernel_libraries;
                   borrows() -> [full names of tensors that other parts own and this one reads too]
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable

import torch


# --------------------------------------------------------------------------
# specs: the data a model is described with
# --------------------------------------------------------------------------
@dataclass(frozen=True)
class ParamSpec:
    shape: tuple
    init: str = "normal"      # 'normal' (std from the writer), 'ones', 'zeros'
    integer: bool = False     # integer tables are kept as int32


@dataclass
class PartSpec:
    kind: str
    args: dict = field(default_factory=dict)
    prefix: str = ""          # joined to the owner's prefix to form tensor names


@dataclass
class LayerSpec:
    block: str                # kind of block, e.g. 'prenorm'
    prefix: str               # e.g. 'model.layers.3.'
    parts: dict               # slot name -> PartSpec


@dataclass(frozen=True)
class ScheduleEntry:
    layer: int                # index into ModelSpec.layers; a layer may be named twice
    cache: int | None = None  # None: a cache of this entry's own; j: read the cache of entry j


@dataclass
class ModelSpec:
    hidden_size: int
    vocab_size: int
    embedding: PartSpec
    layers: list
    schedule: list
    final_norm: PartSpec
    head: PartSpec
    max_positions: int
    eos_token_id: int | tuple | None = None      # the id, or the ids, that end a generation


# --------------------------------------------------------------------------
# registries
# --------------------------------------------------------------------------
class Registry:
    def __init__(self, what: str):
        self.what = what
        self._items: dict[str, type] = {}

    def register(self, kind: str):
        def deco(cls):
            self._items[kind] = cls
            cls.kind = kind
            return cls
        return deco

    def build(self, spec: PartSpec, **extra):
        cls = self._items.get(spec.kind)
        if cls is None:
            raise KeyError(f"no {self.what} of kind '{spec.kind}' is registered "
                           f"(known: {', '.join(sorted(self._items)) or 'none'})")
        return cls(**spec.args, **extra)

    def get(self, kind: str) -> type:
        if kind not in self._items:
            raise KeyError(f"no {self.what} of kind '{kind}' is registered "
                           f"(known: {', '.join(sorted(self._items)) or 'none'})")
        return self._items[kind]

    def __contains__(self, kind):
        return kind in self._items

    def kinds(self):
        return sorted(self._items)


NORMS = Registry("norm")
POSITION_ENCODINGS = Registry("position encoding")
MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
BLOCKS = Registry("block")
EMBEDDINGS = Registry("embedding")
HEADS = Registry("head")


# --------------------------------------------------------------------------
# what a step hands to the parts
# --------------------------------------------------------------------------
@dataclass
class StepContext:
    """One batch of (request, its next tokens), flattened.

    Token t belongs to sequence token_seq[t] (a row of the block tables and of
    slot_ids) and stands at positions[t].  Sequence s owns tokens
    [q_starts[s], q_starts[s+1]) and holds kv_lens[s] positions after the step.
    """
    n_tokens: int
    n_seqs: int
    act_dtype: torch.dtype
    device: torch.device
    token_ids: torch.Tensor            # int32 [T]
    positions: torch.Tensor            # int32 [T]
    token_seq: torch.Tensor            # int32 [T]
    q_starts: list                     # host, n_seqs + 1
    kv_lens: list                      # host, n_seqs
    slot_ids: torch.Tensor             # int32 [n_seqs]
    slots: list                        # host copy
    block_tables: dict                 # group key -> int32 [n_seqs, max_blocks]
    block_size: int
    logit_rows: torch.Tensor | None = None   # int32 [R] token indices whose logits are wanted
    # True while a decode step is recorded for replay (a HIP graph): every sequence brings exactly one
    # token, token t belongs to sequence t, and what changes from replay to replay is only the content
    # of the device tensors above.  The host lists then give the shape alone (kv_lens holds `kv_bound`,
    # which every replay's sequence lengths stay under; `slots` is None): a part must not make device
    # data from them or choose launches by their values.
    recorded: bool = False
    kv_bound: int = 0
    carry: object = None               # what a feed-forward hands on to the next block (its rows, normed), see PreNormBlock
    _memo: dict = field(default_factory=dict)

    def memo(self, key, make: Callable):
        """Per-step data that several layers share (built by the first that asks)."""
        if key not in self._memo:
            self._memo[key] = make()
        return self._memo[key]

    def q_len(self, s: int) -> int:
        return self.q_starts[s + 1] - self.q_starts[s]


@dataclass
class LayerCache:
    """The part of the cache one schedule entry sees."""
    pages: dict                        # name -> [num_pages, *page_shape]
    state: dict                        # name -> [n_slots, *state_shape]
    group: object                      # key into ctx.block_tables (None if the mixer has no pages)
    block_size: int
    writes: bool = True                # False: the pages belong to another entry, read only


# --------------------------------------------------------------------------
# base classes
# --------------------------------------------------------------------------
class Part:
    kernel_libraries: tuple = ()

    def param_specs(self) -> dict:
        return {}

    def load(self, fetch: Callable[[str], torch.Tensor]) -> None:
        """`fetch(local name)` returns the tensor on the device.  Floating tensors come
        in the activation type, except those stored in float32, which stay float32.
        `fetch.shared(full name)` returns a tensor that another part owns and `borrows()` has announced:
        the same memory that its owner gets, uploaded once."""

    def borrows(self) -> list:
        """Full names of tensors that other parts declare and this part reads as well (a head tied to
        the embedding table).  The model checks that someone owns them and uploads each once."""
        return []

    def children(self) -> list:
        """Sub-parts as [(prefix, part)]; a child's tensors are named prefix + its local names."""
        return []


def walk_params(part: "Part", prefix: str = ""):
    """Yields (full tensor name, ParamSpec, owning part, local name) of a part and its children."""
    for local, spec in part.param_specs().items():
        yield prefix + local, spec, part, local
    for child_prefix, child in part.children():
        yield from walk_params(child, prefix + child_prefix)


def walk_parts(part: "Part", prefix: str = ""):
    """Yields (prefix, part) for a part and its children."""
    yield prefix, part
    for child_prefix, child in part.children():
        yield from walk_parts(child, prefix + child_prefix)


class Norm(Part):
    def forward(self, h, ctx: StepContext, rows=None):
        raise NotImplementedError

    def rms_params(self):
        """(weight, eps) if this norm is y = x * rsqrt(mean(x^2) + eps) * weight, which kernels of other parts
        can apply on their way in or leave to the product that follows; None for any other norm (the parts
        then call `forward`)."""
        return None


@dataclass(frozen=True)
class Rotary:
    """A rotation that the kernels apply themselves while they write the cache: pair i of the first
    `rotary_dim` dimensions of every q and k head turns by pos * theta^(-2i/rotary_dim), divided by
    freq_factors[i] if a table is given (float32 [rotary_dim / 2] on the device).  Pairs are
    (i, i + rotary_dim/2), or (2i, 2i+1) when `interleaved`.  rotary_dim 0 rotates nothing."""
    rotary_dim: int
    theta: float
    interleaved: bool = False
    freq_factors: torch.Tensor | None = None


class PositionEncoding(Part):
    def rotary(self) -> "Rotary | None":
        """A `Rotary` if the encoding is one the kernels apply; None if `apply` has to be called."""
        return None

    def apply(self, q, k, ctx: StepContext) -> None:
        raise NotImplementedError


class Mixer(Part):
    window: int | None = None
    graph_safe = False        # True: forward launches the same kernels for every step of one shape (see StepContext.recorded)

    def page_shapes(self, block_size: int) -> dict:
        return {}

    def cache_group(self):
        """(key, window) of the pages this mixer keeps.  Mixers that name the same key share page ids and
        block tables (each has slabs of its own behind them); `window` says how the group's pages age:
        None keeps every position, W gives a page back once all its positions are W or more behind every
        later query.  The key is any hashable value; a mixer whose pages age in a way of its own names a
        key of its own."""
        return (("window", int(self.window)), int(self.window)) if self.window else (("full",), None)

    def state_shapes(self) -> dict:
        return {}

    def forward(self, x, ctx: StepContext, cache: LayerCache, residual) -> None:
        raise NotImplementedError

    # ---- optional: norms fused into the mixer's first kernel (a block asks; the defaults decline) ----
    def forward_from_residual(self, norm: "Norm", ctx: StepContext, cache: LayerCache, residual) -> bool:
        """Apply `norm` to the residual stream inside the mixer's first kernel and run the mixer; False
        (nothing done) if this step or this norm does not allow it, and the block then calls the norm itself."""
        return False

    def takes_scale_later(self, act_dtype) -> bool:
        """Whether `forward` accepts an `ops.ScaleLater` (rows times the norm's weight, the scale still to come) as x."""
        return False


class FeedForward(Part):
    norms_after = False      # True: forward takes then_norm=(norm, scale_later_ok) and may leave norm(residual) in ctx.carry

    def forward(self, x, ctx: StepContext, residual) -> None:
        raise NotImplementedError

    def forward_from_residual(self, norm: "Norm", ctx: StepContext, residual, **more) -> bool:
        """As `Mixer.forward_from_residual`."""
        return False


class Block(Part):
    """A block that sets `chains_norms = True` also has a `first_norm` and takes
    forward(h, ctx, cache, normed=None, then=None): `normed` is first_norm(h) if the block before has made it,
    `then` is (the first norm of the block after, that block's takes_scale_later(dtype)); it returns the
    rows normed by that norm if one of its kernels has made them, else None.  The model passes `normed` and
    `then` only between neighbours that both chain; every other block is called as forward(h, ctx, cache)."""
    mixer: Mixer
    chains_norms = False
    first_norm: "Norm | None" = None

    def takes_scale_later(self, act_dtype) -> bool:
        return False

    def forward(self, h, ctx: StepContext, cache: LayerCache) -> None:
        raise NotImplementedError
