"""Causal grouped-query attention over the paged cache.

Per token (ferrox-models/src/decoder.rs:3224-3560): q, k, v = W x + b, the bias
added before the rotation; q and k rotated by the position encoding; k and v
written into the pages; the query attends to its sequence's pages (its own
position included, through the cache just written); the heads' outputs go
through o_proj (no bias) into the residual stream.  Optionally every head of q
and of k goes through a norm of its own between the bias and the rotation
(`qk_norm`; the reference applies such norms where a model's tensors exist,
decoder.rs:2099-2104, 3256-3267; this architecture has none).
"""
from __future__ import annotations

import math

import torch

from .. import debug, limits, ops
from .base import MIXERS, NORMS, POSITION_ENCODINGS, Mixer, ParamSpec, PartSpec, Rotary
from .linear import Linear, matmul, same_dtype

NO_ROTATION = Rotary(0, 1.0)
EVEN_BLOCKS_PER_CU = 250 / 256     # items of 128 queries pay from about one evenly loaded block per CU on (measured on 256 CUs)


def attention_items(ctx, tile_q: int = 64):
    """Work items of a step, shared by the attention layers of one item size: sequences with one
    new token go to the split decode kernel, the others are cut into blocks of
    tile_q consecutive queries."""
    if ctx.recorded:      # token t is the one token of sequence t; nothing is made from host lists
        return {"n_decode": ctx.n_seqs, "n_tiles": 0, "max_kv": ctx.kv_bound, "dec_seq": ctx.token_seq,
                "dec_tok": ctx.token_seq}
    dec_seq, dec_tok, t_seq, t_tok, t_n = [], [], [], [], []
    max_kv = 1
    for s in range(ctx.n_seqs):
        b, e = ctx.q_starts[s], ctx.q_starts[s + 1]
        if e - b == 1:
            dec_seq.append(s)
            dec_tok.append(b)
            max_kv = max(max_kv, ctx.kv_lens[s])
        else:
            for t0 in range(b, e, tile_q):
                t_seq.append(s)
                t_tok.append(t0)
                t_n.append(min(tile_q, e - t0))
    flat = dec_seq + dec_tok + t_seq + t_tok + t_n
    # through pinned memory, so that the host does not wait here for the kernels launched before
    dev = torch.tensor(flat, dtype=torch.int32).pin_memory().to(ctx.device, non_blocking=True) if flat else None
    nd, nt = len(dec_seq), len(t_seq)
    items = {"n_decode": nd, "n_tiles": nt, "max_kv": max_kv}
    if nd:
        items["dec_seq"], items["dec_tok"] = dev[:nd], dev[nd:2 * nd]
    if nt:
        o = 2 * nd
        items["tile_seq"], items["tile_tok"], items["tile_n"] = dev[o:o + nt], dev[o + nt:o + 2 * nt], dev[o + 2 * nt:]
    return items


@MIXERS.register("paged_attention")
class PagedAttention(Mixer):
    kernel_libraries = ("elementwise", "gemm", "attention")
    graph_safe = True      # its launches depend on device data and on sizes that are fixed per graph

    def __init__(self, hidden_size: int, n_heads: int, n_kv_heads: int, head_dim: int, bias: bool,
                 position: PartSpec, window: int | None = None, scale: float | None = None,
                 qk_norm: PartSpec | None = None):
        """`qk_norm`: kind and arguments of a norm over head_dim; two of them are built, with tensors under
        `q_norm.` and `k_norm.`, and applied to every head of q and of k before the rotation."""
        if n_heads % n_kv_heads:
            raise ValueError(f"n_heads {n_heads} is not a multiple of n_kv_heads {n_kv_heads}")
        if head_dim % limits.HEAD_DIM_STEP or not limits.HEAD_DIM_STEP <= head_dim <= limits.HEAD_DIM_MAX:
            raise ValueError(f"head_dim {head_dim}: the attention kernels take multiples of {limits.HEAD_DIM_STEP} "
                             f"up to {limits.HEAD_DIM_MAX}")
        self.hidden_size, self.n_heads, self.n_kv_heads, self.head_dim = hidden_size, n_heads, n_kv_heads, head_dim
        self.bias = bool(bias)
        self.window = int(window) if window else None
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)   # attention.rs:433
        if not 0.0 < self.scale < math.inf:
            raise ValueError(f"the scale of the attention scores must be positive and finite, got {self.scale}")
        self.position = POSITION_ENCODINGS.build(position)
        self._position_prefix = position.prefix or ""       # where the encoding's own tensors (if any) are named
        self.qw, self.kvw = n_heads * head_dim, n_kv_heads * head_dim
        self.qkv = self.o_proj = None
        self.q_norm = self.k_norm = None
        if qk_norm is not None:
            self.q_norm, self.k_norm = (NORMS.build(PartSpec(qk_norm.kind, dict(qk_norm.args))) for _ in range(2))

    def children(self):
        norms = [("q_norm.", self.q_norm), ("k_norm.", self.k_norm)] if self.q_norm is not None else []
        return [(self._position_prefix, self.position)] + norms

    def param_specs(self):
        H = self.hidden_size
        specs = {"q_proj.weight": ParamSpec((self.qw, H)), "k_proj.weight": ParamSpec((self.kvw, H)),
                 "v_proj.weight": ParamSpec((self.kvw, H)), "o_proj.weight": ParamSpec((H, self.qw))}
        if self.bias:
            specs.update({"q_proj.bias": ParamSpec((self.qw,)), "k_proj.bias": ParamSpec((self.kvw,)),
                          "v_proj.bias": ParamSpec((self.kvw,))})
        return specs

    def load(self, fetch):
        w = torch.cat(same_dtype([fetch("q_proj.weight"), fetch("k_proj.weight"), fetch("v_proj.weight")]), dim=0)
        b = None
        if self.bias:
            b = torch.cat(same_dtype([fetch("q_proj.bias"), fetch("k_proj.bias"), fetch("v_proj.bias")]), dim=0)
        self.qkv = Linear(w, b)
        self.o_proj = Linear(fetch("o_proj.weight"))

    def page_shapes(self, block_size: int) -> dict:
        return {"k": (self.n_kv_heads, block_size, self.head_dim),
                "v": (self.n_kv_heads, self.head_dim, block_size)}

    def forward_from_residual(self, norm, ctx, cache, residual) -> bool:
        """Few tokens: the norm is applied inside the q/k/v product (up to 16 rows it saves a launch; with
        more, every block's reading and norming of all rows costs more than the norm kernel)."""
        rms = norm.rms_params()
        if (ctx.act_dtype != torch.bfloat16 or rms is None or residual.shape[0] > 16 or self.q_norm is not None
                or not ops.can_fuse_norm(residual, self.qkv.weight, residual.shape[0])):
            return False
        debug.region("qkv")
        qkv = ops.gemm(residual, self.qkv.weight, bias=self.qkv.bias, norm=rms)
        self.forward(None, ctx, cache, residual, qkv=qkv)
        return True

    def takes_scale_later(self, act_dtype) -> bool:
        """Whether forward takes an ops.ScaleLater as x (the block before then leaves its rows that way)."""
        w = self.qkv.weight
        return (self.q_norm is None and act_dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and w.shape[1] % 8 == 0
                and w.data_ptr() % 16 == 0)

    def tile_queries(self, ctx, dtype, block_size: int) -> int:
        """Queries per work item of this step's prompt portions: 64, or 128 where the kernel takes that many (a block
        of eight waves then shares every tile of keys it brings in between twice as many queries).  The kernel gives
        a launch of no more blocks than the GPU has CUs (256) two groups of waves per block, which halves a block's chain of
        tiles; so: items of 64 while they number no more than the CUs; else items of 128 if those do (a 2,048-token
        portion deep in a prompt: 603 against 784 us at 16 heads); else items of 128 if they still number about
        one evenly loaded block per CU (blocks of a portion that starts a prompt differ in work up to the portion's
        length in keys and count by their mean share of the longest; +8-26 % from 448 such blocks on); else 64."""
        if ctx.recorded:
            return 64
        widest = ops.attention_tile_queries(dtype, self.head_dim, block_size)
        if widest == 64:
            return 64
        cus = ops.compute_units(ctx.device)
        small = large = 0
        even_blocks = 0.0
        for s in range(ctx.n_seqs):
            n = ctx.q_starts[s + 1] - ctx.q_starts[s]
            if n > 1:
                before = ctx.kv_lens[s] - n
                small += -(-n // 64) * self.n_heads
                large += -(-n // widest) * self.n_heads
                even_blocks += -(-n // widest) * self.n_heads * (before + n / 2) / (before + n)
        if small <= cus:
            return 64
        return widest if large <= cus or even_blocks >= EVEN_BLOCKS_PER_CU * cus else 64

    def normed_heads(self, x, ctx):
        """q [T, qw], k [T, kvw] with every head normed, and v [T, kvw]: the q and k products in float32 (the
        norms read float32 rows), each head a row of a [T * (nh + nkv), head_dim] matrix that the norm kernels
        gather their rows from."""
        T, nh, nkv, hd = ctx.n_tokens, self.n_heads, self.n_kv_heads, self.head_dim
        w, b = self.qkv.weight, self.qkv.bias
        cut = self.qw + self.kvw
        qk = matmul(x, w[:cut], bias=None if b is None else b[:cut], epilogue=ops.EPI_STORE_F32)
        v = matmul(x, w[cut:], bias=None if b is None else b[cut:])

        def head_rows():
            first = torch.arange(T, dtype=torch.int32, device=qk.device)[:, None] * (nh + nkv)
            heads = torch.arange(nh + nkv, dtype=torch.int32, device=qk.device)[None, :]
            rows = first + heads
            return rows[:, :nh].reshape(-1).contiguous(), rows[:, nh:].reshape(-1).contiguous()

        q_rows, k_rows = ctx.memo(f"head rows {nh} {nkv}", head_rows)
        heads = qk.view(T * (nh + nkv), hd)
        q = self.q_norm.forward(heads, ctx, rows=q_rows).view(T, self.qw)
        k = self.k_norm.forward(heads, ctx, rows=k_rows).view(T, self.kvw)
        return q, k, v

    def forward(self, x, ctx, cache, residual, qkv=None) -> None:
        table = ctx.block_tables[cache.group]
        k_pages, v_pages = cache.pages["k"], cache.pages["v"]
        rot = self.position.rotary()
        debug.region("qkv")
        fused = (qkv is None and self.q_norm is None and rot is not None
                 and ops.can_qkv_rope(x, self.qkv.weight, ctx.n_tokens, self.head_dim, rot.rotary_dim, rot.interleaved))
        if fused:
            # few tokens: rotation and cache write happen in the product's epilogue
            qkv = ops.qkv_rope(x, self.qkv.weight, self.qkv.bias, ctx.positions, ctx.token_seq, table,
                               k_pages if cache.writes else None, v_pages if cache.writes else None,
                               self.n_heads, self.n_kv_heads, self.head_dim, cache.block_size, rot.rotary_dim, rot.theta,
                               rot.freq_factors)
            q = qkv[:, :self.qw]
        else:
            if self.q_norm is not None:           # every head of q and k through its norm, between bias and rotation
                q, k, v = self.normed_heads(x, ctx)
                qkv = q
            else:
                if qkv is None:
                    if isinstance(x, ops.ScaleLater):     # rows of a norm whose scale the product applies
                        qkv = ops.gemm(x.x, self.qkv.weight, bias=self.qkv.bias, row_ss=(x.ss, x.eps))
                    else:
                        qkv = self.qkv(x)
                q, k, v = qkv[:, :self.qw], qkv[:, self.qw:self.qw + self.kvw], qkv[:, self.qw + self.kvw:]
            debug.region("rope + cache write")
            if rot is None:
                self.position.apply(q, k, ctx)
                rot = NO_ROTATION
            ops.rope_kv_write(q, k, v, ctx.positions, ctx.token_seq, table,
                              k_pages if cache.writes else None, v_pages if cache.writes else None,
                              self.n_heads, self.n_kv_heads, self.head_dim, cache.block_size, rot.rotary_dim, rot.theta,
                              rot.interleaved, rot.freq_factors)
        debug.region("attention")
        out = torch.empty((ctx.n_tokens, self.qw), dtype=qkv.dtype, device=qkv.device)
        tile_q = ctx.memo(f"attention tile {self.n_heads} {self.head_dim} {cache.block_size} {q.dtype}",
                          lambda: self.tile_queries(ctx, q.dtype, cache.block_size))
        items = ctx.memo(f"attention_items {tile_q}", lambda: attention_items(ctx, tile_q))
        common = (self.n_heads, self.n_kv_heads, self.head_dim, cache.block_size, self.window, self.scale)
        if items["n_tiles"]:
            ops.attention_tiles(q, out, k_pages, v_pages, table, ctx.positions,
                                items["tile_seq"], items["tile_tok"], items["tile_n"], *common, tile_q=tile_q)
        if items["n_decode"]:
            ops.attention_decode(q, out, k_pages, v_pages, table, ctx.positions,
                                 items["dec_seq"], items["dec_tok"], *common, max_kv_len=items["max_kv"])
        debug.region("o_proj")
        self.o_proj(out, epilogue=ops.EPI_RESID, out=residual)
