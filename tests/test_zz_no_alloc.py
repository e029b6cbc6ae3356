"""The decode attention's entry point that allocates nothing (`fx_attn_decode_static`, for callers that cannot
call hipMalloc) against the entry point whose caller brings the buffers for the chunks' partial results
(`fx_attn_decode`): called through ctypes, two calls in a row on one GPU, the second with a smaller input, so
that it runs over what the first left in the library's array."""
import ctypes
import math

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def library():
    from ferrox_amd.csrc.build import load_library
    lib = load_library("attention")
    vp, ci, cl, cf = ctypes.c_void_p, ctypes.c_int, ctypes.c_long, ctypes.c_float
    common = [vp, ci, vp, cl, vp, cl, vp, vp, vp, ci, vp, vp, vp, ci, ci, ci, ci, ci, ci, cf]
    lib.fx_attn_decode.argtypes = common + [vp, vp, ci, ci, ci]
    lib.fx_attn_decode_static.argtypes = common + [ci, ci, ci]
    lib.fx_attn_decode.restype = lib.fx_attn_decode_static.restype = lib.fx_attn_static_init.restype = ci
    lib.fx_attn_static_capacity.restype = cl
    lib.fx_last_error.restype = ctypes.c_char_p
    return lib


def case(dtype, n, nh, nkv, hd, bs, lens, seed):
    """random queries, pages and block tables for n single queries at the ends of sequences of `lens` keys"""
    g = torch.Generator().manual_seed(seed)
    max_blocks = max(-(-L // bs) for L in lens)
    n_pages = n * max_blocks + 3
    table = torch.randperm(n_pages, generator=g)[: n * max_blocks].reshape(n, max_blocks).to(torch.int32).to(DEV)
    q = (torch.randn(n, nh * hd, generator=g) * 0.5).to(dtype).to(DEV)
    k_pages = torch.randn(n_pages, nkv, bs, hd, generator=g).to(dtype).to(DEV)
    v_pages = torch.randn(n_pages, nkv, hd, bs, generator=g).to(dtype).to(DEV)
    positions = torch.tensor([L - 1 for L in lens], dtype=torch.int32, device=DEV)
    items = torch.arange(n, dtype=torch.int32, device=DEV)
    return q, k_pages, v_pages, table, positions, items, max_blocks


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_decode_attention_that_allocates_nothing(dtype):
    lib = library()
    assert lib.fx_attn_static_init() == 0, lib.fx_last_error().decode()
    code = 1 if dtype == torch.bfloat16 else 0
    nh, nkv, hd, bs, window, chunk = 8, 2, 64, 16, 0, 128
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # the second call is smaller in every way: fewer queries, shorter sequences, fewer chunks
    for n, lens, seed in ((6, [700, 3, 129, 512, 640, 77], 1), (2, [200, 65], 2)):
        q, k_pages, v_pages, table, positions, items, max_blocks = case(dtype, n, nh, nkv, hd, bs, lens, seed)
        splits = -(-max(lens) // chunk)
        want, got = torch.zeros_like(q), torch.zeros_like(q)
        part_o = torch.empty(n, nh, splits, hd, dtype=torch.float32, device=DEV)
        part_ml = torch.empty(n, nh, splits, 2, dtype=torch.float32, device=DEV)
        args = (stream, code, p(q), q.stride(0), None, q.stride(0), p(k_pages), p(v_pages), p(table), max_blocks,
                p(positions), p(items), p(items), n, nh, nkv, hd, bs, window, 1.0 / math.sqrt(hd))
        with_out = lambda out: args[:4] + (p(out),) + args[5:]
        assert lib.fx_attn_decode(*with_out(want), p(part_o), p(part_ml), splits, chunk, 0) == 0, lib.fx_last_error().decode()
        torch.cuda.synchronize()
        # torch's counters see only torch's allocator; the driver's free memory sees a hipMalloc inside the library too
        # (the array's address was looked up by fx_attn_static_init above, so nothing is left to set up)
        held = (torch.cuda.memory_allocated(), torch.cuda.memory_reserved())
        free_before = torch.cuda.mem_get_info()[0]
        assert lib.fx_attn_decode_static(*with_out(got), splits, chunk, 0) == 0, lib.fx_last_error().decode()
        torch.cuda.synchronize()
        assert (torch.cuda.memory_allocated(), torch.cuda.memory_reserved()) == held
        assert torch.cuda.mem_get_info()[0] == free_before, "the device's free memory changed across the call"
        assert torch.isfinite(got.float()).all() and float(got.float().abs().max()) > 0
        assert torch.equal(got, want), f"{dtype}, {n} queries: the two entry points differ"
    # more partial results than the array holds: refused with a message, nothing launched
    n, lens = 64, [70000] * 64
    too_many = lib.fx_attn_static_capacity() // (n * nh * (hd + 2)) + 1
    q, k_pages, v_pages, table, positions, items, max_blocks = case(dtype, 2, nh, nkv, hd, bs, [40, 40], 3)
    out = torch.zeros_like(q)
    rc = lib.fx_attn_decode_static(stream, code, p(q), q.stride(0), p(out), q.stride(0), p(k_pages), p(v_pages), p(table),
                                   max_blocks, p(positions), p(items), p(items), n, nh, nkv, hd, bs, window, 0.125,
                                   too_many, 64, 0)
    assert rc != 0 and "more than" in lib.fx_last_error().decode()
    torch.cuda.synchronize()
    assert float(out.float().abs().max()) == 0.0
    # a scale that is not positive is refused by both entry points (the kernels scale a row's maximum once)
    for scale in (0.0, -0.125):
        rc = lib.fx_attn_decode_static(stream, code, p(q), q.stride(0), p(out), q.stride(0), p(k_pages), p(v_pages), p(table),
                                       max_blocks, p(positions), p(items), p(items), 2, nh, nkv, hd, bs, window, scale, 1, 64, 0)
        assert rc != 0 and "scale" in lib.fx_last_error().decode()


def test_static_entry_point_on_a_stream_that_is_captured():
    """under stream capture the call launches the same kernels (recorded, then replayed twice with other work
    between the replays) and gives the bits of the eager call; the array's address was looked up beforehand"""
    lib = library()
    assert lib.fx_attn_static_init() == 0, lib.fx_last_error().decode()
    dtype, code = torch.bfloat16, 1
    nh, nkv, hd, bs, window, chunk = 8, 2, 64, 16, 0, 128
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    lens = [300, 129, 40]
    q, k_pages, v_pages, table, positions, items, max_blocks = case(dtype, 3, nh, nkv, hd, bs, lens, 5)
    splits = -(-max(lens) // chunk)
    want, got = torch.zeros_like(q), torch.zeros_like(q)
    call = lambda stream, out: lib.fx_attn_decode_static(
        ctypes.c_void_p(stream), code, p(q), q.stride(0), p(out), q.stride(0), p(k_pages), p(v_pages), p(table), max_blocks,
        p(positions), p(items), p(items), 3, nh, nkv, hd, bs, window, 1.0 / math.sqrt(hd), splits, chunk, 0)
    assert call(torch.cuda.current_stream().cuda_stream, want) == 0, lib.fx_last_error().decode()
    torch.cuda.synchronize()
    graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        graph.capture_begin()
        try:
            rc = call(side.cuda_stream, got)
        finally:
            graph.capture_end()
    assert rc == 0, lib.fx_last_error().decode()
    torch.cuda.current_stream().wait_stream(side)
    for replay in range(2):
        got.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay {replay}"
        (q.float() @ q.float().T).sum().item()              # other work between the replays
