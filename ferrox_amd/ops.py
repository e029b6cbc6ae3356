"""Python faces of the HIP kernels: argument checks, then one ctypes call.

Tensors live on the GPU; the kernels run on torch's current stream.  There is no
other implementation behind these functions: a tensor on the CPU, or a missing
library, raises.
"""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_long, c_void_p

import math

import torch

from .csrc.build import load_library

FX_F32, FX_BF16 = 0, 1
EPI_STORE, EPI_STORE_F32, EPI_RESID, EPI_GATED = 0, 1, 2, 3
# what the gate of a gated product goes through (EPI_GATED stores activation(gate) * up); ACT_* in csrc/gemm.hip
ACTIVATIONS = {"silu": 0, "gelu_tanh": 1, "gelu": 2, "relu": 3}
GATE_SOFTMAX, GATE_SIGMOID = 0, 1
ROPE_NEOX, ROPE_INTERLEAVED = 0, 1


class KernelError(RuntimeError):
    pass


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float32:
        return FX_F32
    if dt == torch.bfloat16:
        return FX_BF16
    raise KernelError(f"kernels take float32 and bfloat16 tensors, not {dt}")


def _p(t):
    if t is None:
        return None
    if not t.is_cuda:
        raise KernelError("kernel called with a tensor that is not on the GPU")
    return t.data_ptr()           # (a plain integer: ctypes turns it into the pointer argument itself)


# the current stream's handle, asked for before every launch: straight from the runtime's binding where this torch
# has it (a fifth of the host's time per launch went into the Stream object that the public call builds)
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_device_index = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    if _raw_stream is not None and _device_index is not None:
        return _raw_stream(_device_index())
    return torch.cuda.current_stream().cuda_stream


_sigs = {
    ("elementwise", "fx_embed"): [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int],
    ("elementwise", "fx_rmsnorm"): [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_float],
    ("elementwise", "fx_rope_kv_write"): [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int,
                                          c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                          c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p],
    ("elementwise", "fx_residual_add"): [c_void_p, c_int, c_void_p, c_void_p, c_long],
    ("elementwise", "fx_cast"): [c_void_p, c_int, c_void_p, c_int, c_void_p, c_long],
    ("elementwise", "fx_moe_combine"): [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                        c_int, c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p],
    ("elementwise", "fx_fill_u32"): [c_void_p, c_void_p, ctypes.c_uint, c_long],
    ("elementwise", "fx_feed_tokens"): [c_void_p, c_void_p, c_void_p, c_void_p, c_int],
    ("gemm", "fx_gemm"): [c_void_p, c_int, c_int, c_void_p, c_long, c_void_p, c_long, c_long, c_void_p, c_int,
                          c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                          c_void_p, c_int, c_float, c_void_p, c_int, c_int, c_int, c_int, c_long, c_void_p, c_int, c_int],
    ("gemm", "fx_qkv_rope"): [c_void_p, c_void_p, c_long, c_void_p, c_long, c_void_p, c_int, c_void_p, c_long, c_int, c_int,
                              c_void_p, c_int, c_float, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                              c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p],
    ("attention", "fx_attn_tiles"): [c_void_p, c_int, c_void_p, c_long, c_void_p, c_long, c_void_p, c_void_p,
                                     c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                     c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int],
    ("attention", "fx_attn_tile_queries"): [c_int, c_int, c_int],
    ("attention", "fx_attn_decode"): [c_void_p, c_int, c_void_p, c_long, c_void_p, c_long, c_void_p, c_void_p,
                                      c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int,
                                      c_int, c_int, c_int, c_int, c_int, c_float,
                                      c_void_p, c_void_p, c_int, c_int, c_int],
    ("moe", "fx_router_select"): [c_void_p, c_void_p, c_long, c_long, c_int, c_int, c_int, c_int, c_int,
                                  c_void_p, c_void_p, c_void_p],
    ("moe", "fx_router_select_align"): [c_void_p, c_void_p, c_long, c_int, c_int, c_int, c_int, c_int,
                                        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
    ("moe", "fx_moe_front"): [c_void_p, c_void_p, c_long, c_void_p, c_int, c_float, c_void_p, c_void_p, c_int, c_int,
                              c_int, c_int, c_int, c_int, c_int] + [c_void_p] * 9 + [c_int],
    ("moe", "fx_moe_align"): [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int],
    ("sampling", "fx_sample_greedy"): [c_void_p, c_void_p, c_long, c_int, c_int, c_void_p, c_void_p, c_void_p],
    ("sampling", "fx_sample"): [c_void_p, c_void_p, c_long, c_void_p, c_int, c_int] + [c_void_p] * 10,
}
_fns: dict = {}


def _fn(lib: str, name: str):
    key = (lib, name)
    entry = _fns.get(key)
    if entry is None:
        handle = load_library(lib)
        f = getattr(handle, name)
        f.argtypes = _sigs[key]
        f.restype = c_int
        entry = _fns[key] = (f, handle)
    return entry


def _call(lib: str, name: str, *args) -> None:
    f, handle = _fn(lib, name)
    if f(*args):
        raise KernelError(handle.fx_last_error().decode())


def _i32(t, what):
    if t is not None and t.dtype != torch.int32:
        raise KernelError(f"{what} must be int32, got {t.dtype}")
    return t


# ---------------------------------------------------------------------------
def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """h[t] = table[ids[t]] as float32."""
    V, H = table.shape
    T = ids.numel()
    if out is None:
        out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    _call("elementwise", "fx_embed", _stream(), dtype_code(table.dtype), _p(table), _p(_i32(ids, "ids")), _p(out), T, H, V)
    return out


def rmsnorm(h: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
            rows: torch.Tensor | None = None, out: torch.Tensor | None = None) -> torch.Tensor:
    """Rows of float32 `h` (all, or those in `rows`) normed into `out_dtype`."""
    if h.dtype != torch.float32 or not h.is_contiguous():
        raise KernelError("rmsnorm reads a contiguous float32 residual stream")
    H = h.shape[-1]
    if weight.numel() != H:
        raise KernelError(f"rmsnorm weight has {weight.numel()} elements for width {H}")
    R = h.shape[0] if rows is None else rows.numel()
    if out is None:
        out = torch.empty((R, H), dtype=out_dtype, device=h.device)
    _call("elementwise", "fx_rmsnorm", _stream(), dtype_code(out_dtype), _p(h), _p(_i32(rows, "rows")), _p(weight),
          dtype_code(weight.dtype), _p(out), R, H, float(eps))
    return out


def _freq_factors(freq_factors, rotary_dim):
    if freq_factors is None:
        return None
    if freq_factors.dtype != torch.float32 or not freq_factors.is_contiguous() or freq_factors.numel() != rotary_dim // 2:
        raise KernelError(f"rotary frequency factors must be {rotary_dim // 2} contiguous float32 values")
    return freq_factors


_inv_freq_tables: dict = {}


def rotary_frequencies(device, rotary_dim: int, theta: float) -> torch.Tensor | None:
    """float32 [rotary_dim / 2] on the device: theta^(-2i/rotary_dim), worked out in float64 on the host and
    rounded once, so that the numbers do not depend on whose `powf` made them (the reference makes them in
    float32, ferrox-core/src/attention.rs:26: the last bit is its libm's).  The kernels multiply them by the
    position in float32, as the reference does (attention.rs:27).  Tables are kept for the life of the process:
    recorded steps hold their addresses."""
    if rotary_dim <= 0:
        return None
    key = (torch.device(device), int(rotary_dim), float(theta))
    if key not in _inv_freq_tables:
        values = [1.0 / float(theta) ** (2.0 * i / rotary_dim) for i in range(rotary_dim // 2)]
        _inv_freq_tables[key] = torch.tensor(values, dtype=torch.float64).to(torch.float32).to(device)
    return _inv_freq_tables[key]


def rope_kv_write(q, k, v, positions, token_seq, block_table, k_pages, v_pages, n_heads, n_kv_heads,
                  head_dim, block_size, rotary_dim, theta, interleaved=False, freq_factors=None) -> None:
    """Rotate q in place; rotate k and write it and v into the pages (skipped when k_pages is None).
    q, k, v are 2-D views [T, heads*head_dim] with unit inner stride.  `freq_factors` (float32
    [rotary_dim / 2] or None): the angle of pair i is divided by freq_factors[i]."""
    T = q.shape[0]
    freq_factors = _freq_factors(freq_factors, rotary_dim)
    for t in (q, k, v):
        if t.stride(-1) != 1 or t.dtype != q.dtype:
            raise KernelError("rope_kv_write wants q, k, v of one dtype with unit inner stride")
    if k_pages is not None:
        if k_pages.dtype != q.dtype or v_pages.dtype != q.dtype:
            raise KernelError("cache pages and activations differ in dtype")
        if tuple(k_pages.shape[1:]) != (n_kv_heads, block_size, head_dim) or \
                tuple(v_pages.shape[1:]) != (n_kv_heads, head_dim, block_size):
            raise KernelError(f"cache pages have shapes {tuple(k_pages.shape)}, {tuple(v_pages.shape)}; expected "
                              f"[pages,{n_kv_heads},{block_size},{head_dim}] and [pages,{n_kv_heads},{head_dim},{block_size}]")
    _call("elementwise", "fx_rope_kv_write", _stream(), dtype_code(q.dtype), _p(q), q.stride(0), _p(k), k.stride(0),
          _p(v), v.stride(0), _p(_i32(positions, "positions")), _p(_i32(token_seq, "token_seq")),
          _p(_i32(block_table, "block_table")), block_table.shape[1] if block_table is not None else 0,
          _p(k_pages), _p(v_pages), T, n_heads, n_kv_heads, head_dim, block_size, rotary_dim,
          1 if interleaved else 0, _p(rotary_frequencies(q.device, rotary_dim, theta)), _p(freq_factors))


def residual_add(h: torch.Tensor, y: torch.Tensor) -> None:
    """h += y, summed in float32."""
    if h.dtype != torch.float32 or h.shape != y.shape or not h.is_contiguous() or not y.is_contiguous():
        raise KernelError("residual_add wants a contiguous float32 h and a y of the same shape")
    _call("elementwise", "fx_residual_add", _stream(), dtype_code(y.dtype), _p(h), _p(y), h.numel())


def cast(src: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    if src.dtype == dtype:
        return src
    src = src.contiguous()
    dst = torch.empty(src.shape, dtype=dtype, device=src.device)
    _call("elementwise", "fx_cast", _stream(), dtype_code(src.dtype), _p(src), dtype_code(dtype), _p(dst), src.numel())
    return dst


def fill_u32(t: torch.Tensor, value: int = 0) -> None:
    if not t.is_contiguous() or t.element_size() * t.numel() % 4:
        raise KernelError("fill_u32 wants a contiguous buffer of whole 32-bit words")
    _call("elementwise", "fx_fill_u32", _stream(), _p(t), value, t.element_size() * t.numel() // 4)


def feed_tokens(tokens: torch.Tensor, ids: torch.Tensor, pairs: torch.Tensor, n_tokens: int, n_ids: int) -> None:
    """tokens[pairs[i, 0]] = ids[pairs[i, 1]], all int32 on the device.  `pairs` [n, 2] was written by the host,
    which has checked it against `n_tokens` and `n_ids`; the ids come from the sampling kernel."""
    for t, name in ((tokens, "tokens"), (ids, "ids"), (pairs, "pairs")):
        if t.dtype != torch.int32 or not t.is_contiguous() or not t.is_cuda:
            raise KernelError(f"feed_tokens: {name} must be contiguous int32 on the GPU")
    if pairs.dim() != 2 or pairs.shape[1] != 2:
        raise KernelError("feed_tokens: pairs must be [n, 2]")
    if tokens.numel() < n_tokens or ids.numel() < n_ids:
        raise KernelError("feed_tokens: a buffer is shorter than the bound its pairs were checked against")
    _call("elementwise", "fx_feed_tokens", _stream(), _p(tokens), _p(ids), _p(pairs), pairs.shape[0])


class ScaleLater:
    """Rows x = round(h * w) of an RMSNorm whose scale is still to come: `ss` [T, n] holds sums of squares of
    parts of each row of h, and row t is to be scaled by rsqrt(sum(ss[t]) / width + eps).  `gemm(..., row_ss=)`
    applies the scale to its product, which is the rounding of the norm that `gemm(..., norm=)` applies itself."""
    __slots__ = ("x", "ss", "eps")

    def __init__(self, x, ss, eps):
        self.x, self.ss, self.eps = x, ss, eps


def moe_combine(h, y_sorted, inv, weights, top_k, shared=None, gate=None, scale_later=None):
    """h[t] += sum_j weights[t, j] * y_sorted[inv[t*k + j]] (inv None: y is in pair order t*k + j)
    + gate[t] * shared[t] if the float32 output of a shared expert is given; `shared` may also be
    [S, T, H], partial outputs that are summed first.
    `scale_later` = (norm weight, eps, dtype): also returns the new rows as a ScaleLater for that RMSNorm."""
    T, H = h.shape
    if y_sorted.dtype != torch.float32 or h.dtype != torch.float32:
        raise KernelError("moe_combine works on float32")
    slabs = 1
    if shared is not None:
        if shared.dtype != torch.float32 or not shared.is_contiguous() or shared.shape[-2:] != h.shape or shared.dim() > 3:
            raise KernelError("moe_combine: the shared expert's output must be float32 [T, H] or [S, T, H]")
        slabs = shared.shape[0] if shared.dim() == 3 else 1
    x, nw, eps, code, ss = None, None, 0.0, 0, None
    if scale_later is not None:
        nw, eps, dt = scale_later
        if nw.numel() != H or not nw.is_contiguous() or not h.is_contiguous():
            raise KernelError(f"moe_combine: norm weight of {nw.numel()} elements for width {H}")
        x, code = torch.empty((T, H), dtype=dt, device=h.device), dtype_code(dt)
        ss = torch.empty((T, (H + 255) // 256), dtype=torch.float32, device=h.device)
    _call("elementwise", "fx_moe_combine", _stream(), _p(h), _p(y_sorted), _p(_i32(inv, "inv")), _p(weights),
          _p(shared), _p(gate), T, H, top_k, slabs, _p(nw), dtype_code(nw.dtype) if nw is not None else 0,
          _p(x), code, _p(ss))
    return ScaleLater(x, ss, float(eps)) if ss is not None else None


def gemm(a: torch.Tensor, w: torch.Tensor, *, epilogue: int = EPI_STORE, out: torch.Tensor | None = None,
         bias: torch.Tensor | None = None, row_scale: torch.Tensor | None = None,
         a_rows: torch.Tensor | None = None, c_rows: torch.Tensor | None = None,
         expert_offsets: torch.Tensor | None = None,
         n_rows: int | None = None, n_out: int | None = None, up_offset: int = 0,
         norm: tuple | None = None, pair_ids: torch.Tensor | None = None, pair_div: int = 1,
         always: tuple | None = None, w_kblocked: bool = False, row_ss: tuple | None = None,
         activation: str = "silu") -> torch.Tensor:
    """C[m, n] = sum_k a[m, k] * w[n, k] with an epilogue.

    `w` is [N, K], or [E, N, K] with `expert_offsets` [E+1] (rows sorted by expert).
    EPI_STORE stores in a's dtype (+bias); EPI_STORE_F32 stores float32; EPI_RESID adds the
    product (times row_scale[m]) into the float32 `out`; EPI_GATED multiplies two
    matrices (rows [0, n_out) and [up_offset/K, ...) of w) and stores activation(gate) * up,
    `activation` being one of ACTIVATIONS.
    `a_rows` gathers the rows of a; `n_rows` is the number of logical rows then.  `c_rows`
    scatters the rows of the output (row_scale stays indexed by the logical row).
    `pair_ids` (int32, up to 64 entries) replaces the sorted layout for
    few rows: logical row m belongs to expert pair_ids[m], reads row m // pair_div of `a` and
    writes row m of the output; the kernel groups the rows by expert itself.  `always` = (S, T,
    from_a): the last S experts of `w` are taken by each of T rows (a shared expert cut into S
    pieces); piece s writes output rows n_pairs + s*T + t and reads row t of `a` (from_a) or that
    same row of `a`.
    `w_kblocked`: `w` is stored as `to_kblocked` makes it, [.., K/64, N, 64] (bfloat16, K % 64 == 0).
    `norm` = (weight [K], eps): `a` is the float32 residual stream and RMSNorm is applied on the way
    in (bfloat16 weights, EPI_STORE, at most 32 rows; see `can_fuse_norm`).
    `row_ss` = (ss [M, n] float32, eps): row m of the product is scaled by rsqrt(sum(ss[m]) / K + eps)
    before the bias is added (the rows of `a` are a ScaleLater's; plain stored bfloat16 product, M <= 64).
    """
    if row_ss is not None:
        ss = row_ss[0]
        if ss.dtype != torch.float32 or ss.dim() != 2 or not ss.is_contiguous() or ss.shape[0] != a.shape[0]:
            raise KernelError("gemm: row_ss must be a contiguous float32 [rows, parts]")
    if norm is not None:
        if a.dtype != torch.float32 or w.dtype != torch.bfloat16 or epilogue != EPI_STORE:
            raise KernelError("gemm: the fused norm reads float32 rows for a stored bfloat16 product")
        if norm[0].numel() != a.shape[1] or not norm[0].is_contiguous():
            raise KernelError("gemm: the norm's weight does not fit the rows")
    elif a.dtype != w.dtype:
        raise KernelError(f"gemm: activations are {a.dtype}, weights {w.dtype}")
    if a.dim() != 2 or a.stride(1) != 1:
        raise KernelError("gemm: activations must be 2-D with unit inner stride")
    if not w.is_contiguous():
        raise KernelError("gemm: weights must be contiguous")
    K = a.shape[1]
    grouped = expert_offsets is not None or pair_ids is not None
    n_always, always_rows, always_from_a = (int(always[0]), int(always[1]), 1 if always[2] else 0) if always else (0, 0, 0)
    if pair_ids is not None:
        n_rows = pair_ids.numel()
    if w_kblocked:
        if w.dim() != (4 if grouped else 3) or w.shape[-1] != 64 or w.dtype != torch.bfloat16:
            raise KernelError("gemm: weights in slabs must be bfloat16 [(E,) K/64, N, 64]")
        n_w, kw = w.shape[-2], w.shape[-3] * 64
        E, w_stride = (w.shape[0] - n_always, n_w * kw) if grouped else (0, 0)
    elif grouped:
        if w.dim() != 3:
            raise KernelError("gemm: grouped weights must be [E, N, K]")
        E, n_w, kw = w.shape
        E -= n_always
        w_stride = n_w * kw
    else:
        if w.dim() != 2:
            raise KernelError("gemm: weights must be [N, K]")
        E, (n_w, kw), w_stride = 0, w.shape, 0
    if kw != K:
        raise KernelError(f"gemm: inner sizes differ, activations {K}, weights {kw}")
    M = n_rows if n_rows is not None else a.shape[0]
    if activation not in ACTIVATIONS:
        raise KernelError(f"gemm: activation '{activation}' is not one of {sorted(ACTIVATIONS)}")
    if epilogue == EPI_GATED:
        N = n_out if n_out is not None else n_w // 2
        if up_offset == 0:
            up_offset = N * K
        if up_offset // K + N > n_w:
            raise KernelError("gemm: gate/up rows exceed the weight matrix")
    else:
        N = n_out if n_out is not None else n_w
    out_dtype = w.dtype if epilogue in (EPI_STORE, EPI_GATED) else torch.float32
    out_rows = M + n_always * always_rows
    if out is None:
        if epilogue == EPI_RESID:
            raise KernelError("gemm: the residual epilogue needs `out`")
        out = torch.empty((out_rows, N), dtype=out_dtype, device=a.device)
    if out.dtype != out_dtype or out.dim() != 2 or out.stride(1) != 1 or out.shape[0] < out_rows or out.shape[1] < N:
        raise KernelError(f"gemm: output {tuple(out.shape)} {out.dtype} does not fit [{M},{N}] {out_dtype}")
    if bias is not None and bias.numel() != N:
        raise KernelError(f"gemm: bias has {bias.numel()} elements for {N} columns")
    _call("gemm", "fx_gemm", _stream(), dtype_code(w.dtype), epilogue, _p(a), a.stride(0), _p(w), w_stride, up_offset,
          _p(bias), dtype_code(bias.dtype) if bias is not None else 0, _p(out), out.stride(0),
          _p(row_scale), _p(_i32(a_rows, "a_rows")), _p(_i32(c_rows, "c_rows")),
          _p(_i32(expert_offsets, "expert_offsets")), E, M, N, K,
          _p(norm[0]) if norm is not None else None, dtype_code(norm[0].dtype) if norm is not None else 0,
          float(norm[1]) if norm is not None else (float(row_ss[1]) if row_ss is not None else 0.0),
          _p(_i32(pair_ids, "pair_ids")), int(pair_div),
          n_always, always_rows, always_from_a, n_w if w_kblocked else 0,
          _p(row_ss[0]) if row_ss is not None else None, row_ss[0].shape[1] if row_ss is not None else 0,
          ACTIVATIONS[activation])
    return out


def can_qkv_rope(x, w, n_rows: int, head_dim: int, rotary_dim: int, interleaved: bool) -> bool:
    """Whether qkv_rope takes these operands: up to 64 rows of bfloat16 (or a ScaleLater of them), split-half
    rotation, head and rotary dimensions that are multiples of 32, aligned rows."""
    xt = x.x if isinstance(x, ScaleLater) else x
    return (n_rows <= 64 and not interleaved and head_dim % 32 == 0 and rotary_dim % 32 == 0
            and xt.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and w.dim() == 2 and w.is_contiguous()
            and xt.dim() == 2 and xt.stride(1) == 1 and xt.stride(0) % 8 == 0 and xt.shape[1] % 8 == 0
            and xt.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def qkv_rope(x, w, bias, positions, token_seq, block_table, k_pages, v_pages, n_heads, n_kv_heads, head_dim,
             block_size, rotary_dim, theta, freq_factors=None) -> torch.Tensor:
    """The q/k/v product of few tokens with the rotation and the cache write in its epilogue: returns
    [T, (n_heads + 2 n_kv_heads) head_dim] whose query columns are rotated (the others are not written); rotated
    keys and the values go into their pages (k_pages None: nowhere).  The bits are those of `gemm` followed by
    `rope_kv_write`.  `x` may be a ScaleLater."""
    later = x if isinstance(x, ScaleLater) else None
    xt = later.x if later else x
    T, K = xt.shape
    N = (n_heads + 2 * n_kv_heads) * head_dim
    if w.shape != (N, K):
        raise KernelError(f"qkv_rope: weights {tuple(w.shape)} for [{N}, {K}]")
    if bias is not None and bias.numel() != N:
        raise KernelError(f"qkv_rope: bias has {bias.numel()} elements for {N} columns")
    if k_pages is not None:
        if k_pages.dtype != xt.dtype or v_pages.dtype != xt.dtype:
            raise KernelError("cache pages and activations differ in dtype")
        if tuple(k_pages.shape[1:]) != (n_kv_heads, block_size, head_dim) or \
                tuple(v_pages.shape[1:]) != (n_kv_heads, head_dim, block_size):
            raise KernelError(f"cache pages have shapes {tuple(k_pages.shape)}, {tuple(v_pages.shape)}")
    out = torch.empty((T, N), dtype=xt.dtype, device=xt.device)
    _call("gemm", "fx_qkv_rope", _stream(), _p(xt), xt.stride(0), _p(w), 0, _p(bias),
          dtype_code(bias.dtype) if bias is not None else 0, _p(out), out.stride(0), T, K,
          _p(later.ss) if later else None, later.ss.shape[1] if later else 0, float(later.eps) if later else 0.0,
          _p(_i32(positions, "positions")), _p(_i32(token_seq, "token_seq")), _p(_i32(block_table, "block_table")),
          block_table.shape[1] if block_table is not None else 0, _p(k_pages), _p(v_pages),
          n_heads, n_kv_heads, head_dim, block_size, rotary_dim, _p(rotary_frequencies(xt.device, rotary_dim, theta)),
          _p(_freq_factors(freq_factors, rotary_dim)))
    return out


def to_kblocked(w: torch.Tensor) -> torch.Tensor:
    """[.., N, K] -> [.., K/64, N, 64]: 64 k of every row, then the next 64 k of every row.  A tile of
    rows then reads one contiguous stretch of memory per K step instead of a short piece of every
    row, which is what the memory likes when the weights are streamed."""
    *lead, N, K = w.shape
    if K % 64:
        raise KernelError(f"to_kblocked: K={K} is not a multiple of 64")
    return w.reshape(*lead, N, K // 64, 64).transpose(-3, -2).contiguous()


def can_fuse_norm(h: torch.Tensor, w: torch.Tensor, n_rows: int) -> bool:
    """Whether gemm(h, w, norm=...) takes these operands: few rows, bfloat16 weights, aligned rows."""
    return (h.dtype == torch.float32 and w.dtype == torch.bfloat16 and w.dim() == 2 and n_rows <= 32
            and h.shape[1] % 8 == 0 and h.stride(0) % 4 == 0 and h.stride(1) == 1
            and h.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


_compute_units: dict = {}


def compute_units(device) -> int:
    """CUs of the device (asked for once)."""
    key = torch.device(device) if device is not None else torch.device("cuda", torch.cuda.current_device())
    if key not in _compute_units:
        _compute_units[key] = int(torch.cuda.get_device_properties(key).multi_processor_count)
    return _compute_units[key]


def attention_tile_queries(dtype, head_dim: int, block_size: int) -> int:
    """The most consecutive queries of a sequence that one item of attention_tiles may cover at these sizes: 64,
    or 128 where the kernel has a block of eight waves for them."""
    f, _ = _fn("attention", "fx_attn_tile_queries")
    return int(f(dtype_code(dtype), int(head_dim), int(block_size)))


def attention_tiles(q, out, k_pages, v_pages, block_table, positions, item_seq, item_tok, item_n,
                    n_heads, n_kv_heads, head_dim, block_size, window, scale, tile_q: int = 64) -> None:
    """Blocks of queries: item i is item_n[i] <= tile_q consecutive tokens of sequence item_seq[i] from token
    item_tok[i] on; tile_q is 64 or attention_tile_queries(...)."""
    _call("attention", "fx_attn_tiles", _stream(), dtype_code(q.dtype), _p(q), q.stride(0), _p(out), out.stride(0),
          _p(k_pages), _p(v_pages), _p(_i32(block_table, "block_table")), block_table.shape[1],
          _p(_i32(positions, "positions")), _p(_i32(item_seq, "item_seq")), _p(_i32(item_tok, "item_tok")),
          _p(_i32(item_n, "item_n")), item_seq.numel(), n_heads, n_kv_heads, head_dim, block_size,
          int(window or 0), float(scale), int(tile_q))


SPLIT_PARTIAL_ROUNDS = True      # decode attention: more chunks where the blocks' last round over the CUs would be far from full


def decode_attention_chunk(n_items: int, n_heads: int, n_kv_heads: int, max_kv_len: int, cus: int) -> int:
    """Keys per chunk of the bfloat16 decode attention, where the caller names none: the fewest chunks that still put
    about eight waves on every CU (one chunk, and no merge launch, from as many (sequence, kv head) pairs as CUs
    on), unless the waves' last round over the CUs would be far from full."""
    pairs = n_items * n_kv_heads * (-(-(n_heads // n_kv_heads) // 16))
    want = max(1, 8 * cus // max(1, pairs * 8))
    # More (sequence, kv head) pairs than CUs: a CU holds eight waves of this kernel, which the launch groups
    # into blocks of eight or four (one chunk a sequence), so the waves run in rounds, and a last round that
    # is far from full (272 blocks of eight waves on 256 CUs: 17 sequences of 16 kv heads) costs nearly as much
    # as a full one.  Eight chunks a sequence, which the launch then gives to blocks of one wave, fill the CUs
    # evenly: 17 sequences at 2,060 keys 80 -> 58 us, 24 sequences 81 -> 77 us, 36 sequences 125 -> 108 us, 17 at
    # 8,200 keys 285 -> 192 us; where the last round is full (32, 64 sequences) one chunk is 2-4 % ahead, and
    # from four pairs a CU on one chunk is level with every other choice.
    if SPLIT_PARTIAL_ROUNDS and cus < pairs <= 4 * cus and max_kv_len >= 1024:
        per_block = 8                   # waves, as fx_attn_decode picks them for one chunk a sequence
        while per_block > 4 and pairs * (per_block // 2) >= 8 * cus:
            per_block //= 2
        rounds = pairs * per_block / (8 * cus)
        if (math.ceil(rounds) - rounds) / math.ceil(rounds) >= 0.10:
            want = 8
    return max(64, -(-(-(-max_kv_len // want)) // 64) * 64)


def attention_decode(q, out, k_pages, v_pages, block_table, positions, item_seq, item_tok,
                     n_heads, n_kv_heads, head_dim, block_size, window, scale, max_kv_len, chunk=None,
                     waves=0) -> None:
    """Single queries.  The keys go to ceil(max_kv_len / chunk) blocks whose results are merged in ascending
    order.  float32 cuts them at multiples of `chunk`, 256 by default (so that a result does not depend on the
    batch); bfloat16, whose blocks of up to eight waves share a chunk, cuts every sequence's own range of keys (from
    its window's first key to its position) into that many equal chunks of whole tiles of 64, `chunk` by default as
    `decode_attention_chunk` picks it.  `waves`: waves per block, 0 for the launch's own choice."""
    n = item_seq.numel()
    if chunk is None:
        chunk = 256
        if q.dtype == torch.bfloat16:
            chunk = decode_attention_chunk(n, n_heads, n_kv_heads, max_kv_len, compute_units(q.device))
    splits = max(1, -(-max_kv_len // chunk))
    part_o = torch.empty((n, n_heads, splits, head_dim), dtype=torch.float32, device=q.device)
    part_ml = torch.empty((n, n_heads, splits, 2), dtype=torch.float32, device=q.device)
    _call("attention", "fx_attn_decode", _stream(), dtype_code(q.dtype), _p(q), q.stride(0), _p(out), out.stride(0),
          _p(k_pages), _p(v_pages), _p(_i32(block_table, "block_table")), block_table.shape[1],
          _p(_i32(positions, "positions")), _p(_i32(item_seq, "item_seq")), _p(_i32(item_tok, "item_tok")), n,
          n_heads, n_kv_heads, head_dim, block_size, int(window or 0), float(scale),
          _p(part_o), _p(part_ml), splits, chunk, int(waves))


def router_select(logits, n_experts, top_k, renorm, gating=GATE_SOFTMAX, has_gate=False):
    """From float32 router logits [T, >= E (+1)] (any strides, so also the transpose of an
    [E (+1), T] product): (ids int32 [T,k], weights float32 [T,k], gate float32 [T] =
    sigmoid(logits[:, E]) or None)."""
    if logits.dtype != torch.float32 or logits.dim() != 2 or min(logits.stride()) < 1:
        raise KernelError("router_select: logits must be a float32 [T, E] matrix")
    T = logits.shape[0]
    ids = torch.empty((T, top_k), dtype=torch.int32, device=logits.device)
    weights = torch.empty((T, top_k), dtype=torch.float32, device=logits.device)
    gate = torch.empty((T,), dtype=torch.float32, device=logits.device) if has_gate else None
    if logits.shape[1] < n_experts + (1 if has_gate else 0):
        raise KernelError(f"router_select: {logits.shape[1]} columns for {n_experts} experts")
    _call("moe", "fx_router_select", _stream(), _p(logits), logits.stride(0), logits.stride(1), T, n_experts, top_k,
          1 if renorm else 0, gating, _p(ids), _p(weights), _p(gate))
    return ids, weights, gate


def route(logits, n_experts, top_k, renorm, gating=GATE_SOFTMAX, has_gate=False):
    """router_select followed by moe_align; one launch when the batch is small.
    Returns (ids, weights, gate, expert_offsets, sorted_token, sorted_pair, inv)."""
    if logits.dtype != torch.float32 or logits.dim() != 2:
        raise KernelError("route: logits must be a float32 [T, E] matrix")
    T = logits.shape[0]
    dev = logits.device
    if T <= 16 and logits.stride(1) == 1 and logits.shape[1] >= n_experts + (1 if has_gate else 0):
        n = T * top_k
        ids = torch.empty((T, top_k), dtype=torch.int32, device=dev)
        weights = torch.empty((T, top_k), dtype=torch.float32, device=dev)
        gate = torch.empty((T,), dtype=torch.float32, device=dev) if has_gate else None
        offsets = torch.empty((n_experts + 1,), dtype=torch.int32, device=dev)
        buf = torch.empty((3, n), dtype=torch.int32, device=dev)
        f, handle = _fn("moe", "fx_router_select_align")
        rc = f(_stream(), _p(logits), logits.stride(0), T, n_experts, top_k, 1 if renorm else 0, gating, _p(ids),
               _p(weights), _p(gate), _p(offsets), _p(buf[0]), _p(buf[1]), _p(buf[2]))
        if rc == 0:
            return ids, weights, gate, offsets, buf[0], buf[1], buf[2]
        if rc != 2:
            raise KernelError(handle.fx_last_error().decode())
    ids, weights, gate = router_select(logits, n_experts, top_k, renorm, gating, has_gate)
    return (ids, weights, gate) + moe_align(ids, n_experts)


_counters: dict = {}


def _counter(device, n: int = 1) -> torch.Tensor:
    """At least n zeroed words for kernels whose last block finishes the work; a kernel leaves its
    words at zero, so launches that follow each other on a stream share them.  Buffers are never
    freed: a recorded graph may hold their address."""
    key = torch.device(device)
    if key.index is None:
        key = torch.device(key.type, torch.cuda.current_device())
    held = _counters.setdefault(key, [])
    if not held or held[-1].numel() < n:
        held.append(torch.zeros(max(1024, 2 * n), dtype=torch.int32, device=key))
    return held[-1]


def moe_front(h, norm_weight, eps, router, n_experts, top_k, renorm, gating=GATE_SOFTMAX, has_gate=False,
              align: int | None = None):
    """For up to 256 rows of the float32 residual stream, in one launch: RMSNorm into bfloat16, router
    products and selection.  Returns None for sizes the kernel does not take, else
    (x, ids, weights, gate, aligned).  `align` = S asks the same launch for what `moe_align(ids, n_experts,
    always=S)` returns (its last block sorts the pairs): `aligned`, else None."""
    T, H = h.shape
    if (T > 256 or h.dtype != torch.float32 or h.stride(1) != 1 or router.dtype != torch.bfloat16
            or not router.is_contiguous() or router.shape != (n_experts + (1 if has_gate else 0), H)
            or norm_weight.numel() != H):
        return None
    dev = h.device
    x = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
    ids = torch.empty((T, top_k), dtype=torch.int32, device=dev)
    weights = torch.empty((T, top_k), dtype=torch.float32, device=dev)
    gate = torch.empty((T,), dtype=torch.float32, device=dev) if has_gate else None
    logits = torch.empty((T, router.shape[0]), dtype=torch.float32, device=dev)
    offsets = buf = None
    if align is not None:
        offsets = torch.empty((n_experts + 1 + align,), dtype=torch.int32, device=dev)
        buf = torch.empty((3, T * top_k + align * T), dtype=torch.int32, device=dev)
    f, handle = _fn("moe", "fx_moe_front")
    rc = f(_stream(), _p(h), h.stride(0), _p(norm_weight), dtype_code(norm_weight.dtype), float(eps), _p(x), _p(router),
           H, T, n_experts, 1 if has_gate else 0, top_k, 1 if renorm else 0, gating, _p(logits), _p(ids), _p(weights),
           _p(gate), _p(_counter(dev, T + 1)), _p(offsets), _p(buf[0]) if buf is not None else None,
           _p(buf[1]) if buf is not None else None, _p(buf[2]) if buf is not None else None, int(align or 0))
    if rc == 2 and align is not None:      # the sort's counters do not fit beside the front's: without it
        return moe_front(h, norm_weight, eps, router, n_experts, top_k, renorm, gating, has_gate)
    if rc == 2:
        return None
    if rc:
        raise KernelError(handle.fx_last_error().decode())
    return x, ids, weights, gate, (offsets, buf[0], buf[1], buf[2]) if buf is not None else None


def moe_align(ids: torch.Tensor, n_experts: int, always: int = 0):
    """For ids [T, k]: (expert_offsets [E+1], sorted_token [n], sorted_pair [n], inv [n]): sorted row i
    belongs to pair sorted_pair[i] = t*k + j of token sorted_token[i]; inv is the inverse map.
    `always` = S: S further experts follow that every token takes (a shared expert cut into pieces): the
    offsets have E+1+S entries and the sorted arrays n + S*T, piece s owning rows n + s*T + t (token t), whose
    output rows have the same numbers (up to 2048 pairs)."""
    T, k = ids.shape
    n = T * k
    dev = ids.device
    offsets = torch.empty((n_experts + 1 + always,), dtype=torch.int32, device=dev)
    buf = torch.empty((3, n + always * T), dtype=torch.int32, device=dev)
    # many pairs are sorted by many blocks, which hand each other the counts of every group of 64 pairs
    gcnt = torch.empty((-(-n // 64), n_experts), dtype=torch.int32, device=dev) if n > 2048 else None
    _call("moe", "fx_moe_align", _stream(), _p(_i32(ids, "ids")), n, k, n_experts, _p(offsets), _p(buf[0]), _p(buf[1]),
          _p(buf[2]), _p(gcnt), int(always))
    return offsets, buf[0], buf[1], buf[2]


def sample(logits: torch.Tensor, *, temperature=None, draw=None, top_k=None, top_p=None, rep_penalty=None,
           presence=None, frequency=None, hist=None, hist_start=None) -> torch.Tensor:
    """One token per row of float32 logits [R, V]; all per-row parameters are device tensors or None
    (None: greedy / option off)."""
    if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("sample: logits must be float32 [R, V] with unit inner stride")
    R, V = logits.shape
    out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    if temperature is None and hist is None:      # plain greedy: many blocks per row
        part = torch.empty((R, 64, 2), dtype=torch.int32, device=logits.device)
        _call("sampling", "fx_sample_greedy", _stream(), _p(logits), logits.stride(0), R, V, _p(part),
              _p(_counter(logits.device, R)), _p(out))
        return out
    work = torch.empty((R, V), dtype=torch.float32, device=logits.device)
    _call("sampling", "fx_sample", _stream(), _p(logits), logits.stride(0), _p(work), R, V,
          _p(temperature), _p(_i32(top_k, "top_k")), _p(top_p), _p(rep_penalty), _p(presence), _p(frequency),
          _p(draw), _p(_i32(hist, "hist")), _p(_i32(hist_start, "hist_start")), _p(out))
    return out
