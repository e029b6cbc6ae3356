"""Each kernel alone against a plain float64 reference, at sizes other than the engine's."""
import math
import random

import pytest
import torch

import plain_qwen2moe as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def rnd(*shape, dtype=torch.float32, scale=1.0, seed=0):
    g = torch.Generator().manual_seed(seed + sum(shape))
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def close(got, want, dtype, what, k=1):
    """float32: rounding of sums of k products; bfloat16: inputs are exact, the output is rounded once."""
    got, want = got.double().cpu(), want.double().cpu()
    scale = float(want.abs().max()) + 1e-30
    tol = (1e-5 if dtype == torch.float32 else 1e-2) * scale
    err = float((got - want).abs().max())
    assert err <= tol, f"{what}: max error {err:.3e} > {tol:.3e} (scale {scale:.3e})"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(1, 48, 64), (5, 100, 96), (16, 256, 128), (17, 257, 200), (33, 72, 40),
                                    (64, 64, 64), (130, 300, 520), (257, 129, 1032), (3, 50, 100),
                                    (130, 300, 512), (257, 129, 1024), (300, 520, 64), (513, 72, 128), (65, 16, 192),
                                    (40, 65600, 64), (64, 65536, 128), (128, 2048, 2048), (256, 3584, 512), (200, 96, 264),
                                    (256, 4200, 64)])
def test_gemm_plain_and_epilogues(dtype, M, N, K):
    from ferrox_amd import ops
    a, w = rnd(M, K, dtype=dtype), rnd(N, K, dtype=dtype, seed=1)
    bias = rnd(N, dtype=dtype, seed=2)
    ref = a.double() @ w.double().T
    close(ops.gemm(a, w), ref, dtype, "store")
    close(ops.gemm(a, w, bias=bias), ref + bias.double(), dtype, "store+bias")
    close(ops.gemm(a, w, epilogue=ops.EPI_STORE_F32, bias=bias), ref + bias.double(), torch.float32 if dtype == torch.float32 else dtype, "f32 store")
    h = rnd(M, N, seed=3)
    h0 = h.clone()
    scale = rnd(M, seed=4)
    ops.gemm(a, w, epilogue=ops.EPI_RESID, out=h, row_scale=scale)
    close(h, h0.double() + ref * scale.double()[:, None], dtype, "residual")


@pytest.mark.parametrize("T,H,N,k,S", [(1, 2048, 6144, 4, 4), (8, 2048, 6144, 4, 4), (16, 264, 100, 3, 0), (5, 520, 72, 1, 2)])
def test_combine_that_leaves_the_scale_to_the_product(T, H, N, k, S):
    """combine -> rows times the norm's weight and sums of squares -> product that scales its rows,
    against combine -> norm kernel -> product and against the plain formulas"""
    from ferrox_amd import ops
    h = rnd(T, H, scale=2.0)
    y, wts = rnd(T * k, H, seed=1), torch.rand(T, k, generator=torch.Generator().manual_seed(2)).to(DEV)
    shared = rnd(S, T, H, seed=3) if S else None
    gate = torch.rand(T, generator=torch.Generator().manual_seed(4)).to(DEV) if S else None
    gamma = (1.0 + rnd(H, seed=5, scale=0.2)).to(torch.bfloat16)
    w, bias = rnd(N, H, dtype=torch.bfloat16, seed=6, scale=0.05), rnd(N, dtype=torch.bfloat16, seed=7)
    h1, h2 = h.clone(), h.clone()
    ops.moe_combine(h1, y, None, wts, k, shared=shared, gate=gate)
    two = ops.gemm(ops.rmsnorm(h1, gamma, 1e-6, torch.bfloat16), w, bias=bias)
    later = ops.moe_combine(h2, y, None, wts, k, shared=shared, gate=gate, scale_later=(gamma, 1e-6, torch.bfloat16))
    assert isinstance(later, ops.ScaleLater) and torch.equal(h1, h2)
    close(later.ss.sum(1), (h1.double() ** 2).sum(1), torch.float32, "sums of squares")
    got = ops.gemm(later.x, w, bias=bias, row_ss=(later.ss, later.eps))
    want = plain.rms_norm(h1.double().cpu(), gamma.double().cpu(), 1e-6) @ w.double().cpu().T + bias.double().cpu()
    close(got, want, torch.bfloat16, "product with the scale applied afterwards")
    close(two, want, torch.bfloat16, "norm, then product")


@pytest.mark.parametrize("T,H,k,S,sorted_rows", [(130, 2048, 4, 4, False), (300, 1000, 3, 0, True), (140, 2052, 2, 1, True)])
def test_combine_of_many_rows_equals_that_of_few(T, H, k, S, sorted_rows):
    """Many rows go four columns to a thread, few rows one: the same bits in the residual stream and in the rows
    for the next norm, the same sums of squares up to the order of their terms."""
    from ferrox_amd import ops
    assert T * H >= 1 << 18 and (T // 2 + 1) * H < 1 << 18
    h = rnd(T, H, scale=2.0)
    y, wts = rnd(T * k, H, seed=1), torch.rand(T, k, generator=torch.Generator().manual_seed(2)).to(DEV)
    inv = torch.randperm(T * k, generator=torch.Generator().manual_seed(3)).to(torch.int32).to(DEV) if sorted_rows else None
    shared = rnd(S, T, H, seed=3) if S else None
    gate = torch.rand(T, generator=torch.Generator().manual_seed(4)).to(DEV) if S else None
    gamma = (1.0 + rnd(H, seed=5, scale=0.2)).to(torch.bfloat16)
    h_all = h.clone()
    all_rows = ops.moe_combine(h_all, y, inv, wts, k, shared=shared, gate=gate, scale_later=(gamma, 1e-6, torch.bfloat16))
    cut = T // 2
    for lo, hi in ((0, cut), (cut, T)):
        h_part = h[lo:hi].clone()
        part = ops.moe_combine(h_part, y if inv is not None else y[lo * k:hi * k], inv[lo * k:hi * k] if inv is not None else None,
                               wts[lo:hi].contiguous(), k, shared=shared[:, lo:hi].contiguous() if S else None,
                               gate=gate[lo:hi].contiguous() if S else None, scale_later=(gamma, 1e-6, torch.bfloat16))
        assert torch.equal(h_all[lo:hi], h_part), "residual stream"
        assert torch.equal(all_rows.x[lo:hi], part.x), "rows for the next norm"
        close(all_rows.ss[lo:hi], part.ss, torch.float32, "sums of squares per 256 columns")
    want = h.double().cpu() + (wts.double().cpu()[:, :, None] * (y.double().cpu()[inv.long().cpu()] if inv is not None else y.double().cpu()).view(T, k, H)).sum(1)
    if S:
        want = want + gate.double().cpu()[:, None] * shared.double().cpu().sum(0)
    close(h_all, want, torch.float32, "combined rows")


@pytest.mark.parametrize("tile", [256, 192, 128, 64, 12, 4])      # 12, 4: tiles of 192 and of 64 rows x 256 weight rows
@pytest.mark.parametrize("M,N,K", [(300, 400, 192), (513, 200, 64), (70, 520, 448)])
def test_gemm_every_wide_tile(tile, M, N, K):
    """The many-row kernel picks its tile by the sizes; here each tile shape is made to run the same products."""
    from ferrox_amd import debug, ops
    dtype = torch.bfloat16
    a, w, bias = rnd(M, K, dtype=dtype), rnd(N, K, dtype=dtype, seed=1), rnd(N, dtype=dtype, seed=2)
    ref = a.double() @ w.double().T
    h = rnd(M, N, seed=3)
    h0 = h.clone()
    with debug.kernel_switch("gemm", "wide", tile):
        got = ops.gemm(a, w, bias=bias)
        ops.gemm(a, w, epilogue=ops.EPI_RESID, out=h)
        w2 = rnd(2 * N, K, dtype=dtype, seed=4, scale=0.5)
        act = ops.gemm(a, w2, epilogue=ops.EPI_GATED)
    close(got, ref + bias.double(), dtype, "store+bias")
    close(h, h0.double() + ref, dtype, "residual")
    close(act, plain.silu(a.double() @ w2[:N].double().T) * (a.double() @ w2[N:].double().T), dtype, "silu(gate)*up")


@pytest.mark.parametrize("tile", [12, 256, 4])
def test_grouped_gemm_tiles_agree(tile):
    """An expert's rows in tiles of 192 (weights three steps deep), of 256 and of 64 (weights four steps deep) give
    the same sums."""
    from ferrox_amd import debug, ops
    T, E, k, I, H = 900, 6, 2, 64, 256
    x = rnd(T, H, dtype=torch.bfloat16)
    w_gu = rnd(E, 2 * I, H, dtype=torch.bfloat16, seed=1, scale=0.3)
    g = torch.Generator().manual_seed(7)
    # uneven shares: expert 0 gets a third of all pairs, more than one tile of either kind
    first = torch.where(torch.rand(T, generator=g) < 0.66, 0, 1)
    ids = torch.stack([first, 2 + torch.randint(0, E - 2, (T,), generator=g)], dim=1).to(torch.int32).to(DEV)
    offsets, sorted_token, sorted_pair, inv = ops.moe_align(ids, E)
    with debug.kernel_switch("gemm", "wide", tile):
        act = ops.gemm(x, w_gu, epilogue=ops.EPI_GATED, a_rows=sorted_token, expert_offsets=offsets, n_rows=T * k)
    xs = x.double()[sorted_token.long()]
    off = offsets.cpu().tolist()
    assert off[1] - off[0] > 256
    for e in range(E):
        r = slice(off[e], off[e + 1])
        want = plain.silu(xs[r] @ w_gu[e, :I].double().T) * (xs[r] @ w_gu[e, I:].double().T)
        close(act[r], want, torch.bfloat16, f"expert {e}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,I,K", [(1, 32, 64), (7, 48, 96), (40, 100, 72), (200, 176, 256), (300, 100, 128),
                                    (257, 129, 64)])
def test_gemm_gate_up(dtype, M, I, K):
    from ferrox_amd import ops
    a, w = rnd(M, K, dtype=dtype), rnd(2 * I, K, dtype=dtype, seed=1, scale=0.5)
    g, u = a.double() @ w[:I].double().T, a.double() @ w[I:].double().T
    close(ops.gemm(a, w, epilogue=ops.EPI_GATED), plain.silu(g) * u, dtype, "silu(gate)*up")
    # the gate's activation is a parameter of the call: every kernel that has the epilogue takes every activation
    others = {"gelu_tanh": lambda z: 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3))),
              "gelu": lambda z: 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0))), "relu": lambda z: z.clamp(min=0.0),
              "silu": plain.silu}
    assert set(others) == set(ops.ACTIVATIONS)
    for name, f in others.items():
        close(ops.gemm(a, w, epilogue=ops.EPI_GATED, activation=name), f(g) * u, dtype, f"{name}(gate)*up")
    with pytest.raises(ops.KernelError, match="activation"):
        ops.gemm(a, w, epilogue=ops.EPI_GATED, activation="swish2")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,E,k,I,H", [(1, 4, 2, 32, 64), (9, 6, 3, 48, 96), (70, 5, 1, 40, 120), (300, 8, 2, 64, 128),
                                        (64, 3, 2, 24, 72), (520, 4, 3, 128, 256), (700, 3, 2, 200, 192),
                                        (330, 4, 2, 128, 320), (1300, 16, 2, 64, 192)])
def test_grouped_gemm_and_routing_buffers(dtype, T, E, k, I, H):
    """router ids -> align -> grouped gate/up -> grouped down -> combine, against per-token loops."""
    from ferrox_amd import ops
    x = rnd(T, H, dtype=dtype)
    w_gu, w_dn = rnd(E, 2 * I, H, dtype=dtype, seed=1, scale=0.3), rnd(E, H, I, dtype=dtype, seed=2, scale=0.3)
    g = torch.Generator().manual_seed(5)
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32).to(DEV)
    wts = torch.rand(T, k, generator=g).to(DEV)
    offsets, sorted_token, sorted_pair, inv = ops.moe_align(ids, E)
    # the sort: offsets are the counts' prefix sums; every pair sits in its expert's range; order is stable
    counts = torch.bincount(ids.flatten().long().cpu(), minlength=E)
    assert offsets.cpu().tolist() == [0] + torch.cumsum(counts, 0).tolist()
    inv_c, st_c, ids_c = inv.cpu(), sorted_token.cpu(), ids.cpu()
    assert sorted(inv_c.tolist()) == list(range(T * k))
    for i in range(T * k):
        e = int(ids_c.flatten()[i])
        assert offsets[e] <= inv_c[i] < offsets[e + 1] and st_c[inv_c[i]] == i // k and sorted_pair[inv_c[i]] == i
    for e in range(E):
        seg = [i for i in range(T * k) if int(ids_c.flatten()[i]) == e]
        assert [int(inv_c[i]) for i in seg] == list(range(int(offsets[e]), int(offsets[e + 1])))
    act = ops.gemm(x, w_gu, epilogue=ops.EPI_GATED, a_rows=sorted_token, expert_offsets=offsets, n_rows=T * k)
    y = ops.gemm(act, w_dn, epilogue=ops.EPI_STORE_F32, expert_offsets=offsets)
    h = torch.zeros(T, H, device=DEV)
    ops.moe_combine(h, y, inv, wts, k)
    # the same with the second product scattering its rows back into pair order
    y2 = ops.gemm(act, w_dn, epilogue=ops.EPI_STORE_F32, expert_offsets=offsets, c_rows=sorted_pair)
    h2 = torch.zeros(T, H, device=DEV)
    ops.moe_combine(h2, y2, None, wts, k)
    assert torch.equal(h, h2)
    ref = torch.zeros(T, H, dtype=torch.float64)
    xd, gud, dnd = x.double().cpu(), w_gu.double().cpu(), w_dn.double().cpu()
    for t in range(T):
        for j in range(k):
            e = int(ids_c[t, j])
            a = plain.silu(xd[t] @ gud[e, :I].T) * (xd[t] @ gud[e, I:].T)
            if dtype == torch.bfloat16:
                a = a.to(torch.bfloat16).double()       # the engine stores the activation in bfloat16
            ref[t] += float(wts[t, j]) * (a @ dnd[e].T)
    close(h, ref, dtype, "moe")


@pytest.mark.parametrize("T,E,k,I,H", [(1, 4, 2, 32, 64), (8, 60, 4, 1408, 2048), (16, 60, 4, 176, 256), (16, 5, 4, 48, 96),
                                        (3, 700, 8, 64, 128), (7, 1, 1, 40, 72)])
def test_grouped_gemm_from_unsorted_pairs(T, E, k, I, H):
    """few rows: the products group the (token, slot) pairs by expert themselves; same numbers as
    the sorted layout gives, row for row"""
    from ferrox_amd import ops
    dtype = torch.bfloat16
    x = rnd(T, H, dtype=dtype)
    w_gu, w_dn = rnd(E, 2 * I, H, dtype=dtype, seed=1, scale=0.3), rnd(E, H, I, dtype=dtype, seed=2, scale=0.3)
    g = torch.Generator().manual_seed(11)
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32).to(DEV)
    if T >= 8 and E >= 8:
        ids[:, 0] = 5            # one expert with a row of every token
    offsets, sorted_token, sorted_pair, inv = ops.moe_align(ids, E)
    act_s = ops.gemm(x, w_gu, epilogue=ops.EPI_GATED, a_rows=sorted_token, expert_offsets=offsets, n_rows=T * k)
    y_s = ops.gemm(act_s, w_dn, epilogue=ops.EPI_STORE_F32, expert_offsets=offsets, c_rows=sorted_pair)
    act_p = ops.gemm(x, w_gu, epilogue=ops.EPI_GATED, pair_ids=ids, pair_div=k)
    y_p = ops.gemm(act_p, w_dn, epilogue=ops.EPI_STORE_F32, pair_ids=ids)
    assert torch.equal(act_p, act_s[inv.long()])
    assert torch.equal(y_p, y_s)
    xd, gud, dnd = x.double().cpu(), w_gu.double().cpu(), w_dn.double().cpu()
    for t in range(T):
        for j in range(k):
            e = int(ids[t, j])
            a = (plain.silu(xd[t] @ gud[e, :I].T) * (xd[t] @ gud[e, I:].T)).to(torch.bfloat16).double()
            close(y_p[t * k + j], a @ dnd[e].T, dtype, f"pair ({t}, {j})")


@pytest.mark.parametrize("T,E,k,I,H,S", [(1, 4, 2, 32, 64, 1), (8, 60, 4, 1408, 2048, 4), (16, 6, 3, 48, 96, 2), (5, 3, 1, 40, 72, 3)])
def test_shared_expert_as_pieces_beside_unsorted_pairs(T, E, k, I, H, S):
    """a shared expert of width S*I cut into S pieces that every token takes, in the same two launches
    as the routed experts: the combine gives routed + gate * shared"""
    from ferrox_amd import ops
    dtype = torch.bfloat16
    x = rnd(T, H, dtype=dtype)
    w_gu, w_dn = rnd(E, 2 * I, H, dtype=dtype, seed=1, scale=0.3), rnd(E, H, I, dtype=dtype, seed=2, scale=0.3)
    sg, su = rnd(S * I, H, dtype=dtype, seed=3, scale=0.3), rnd(S * I, H, dtype=dtype, seed=4, scale=0.3)
    sd = rnd(H, S * I, dtype=dtype, seed=5, scale=0.3)
    gu_all = torch.cat([w_gu] + [torch.cat([sg[s * I:(s + 1) * I], su[s * I:(s + 1) * I]])[None] for s in range(S)]).contiguous()
    dn_all = torch.cat([w_dn] + [sd[:, s * I:(s + 1) * I][None] for s in range(S)]).contiguous()
    g = torch.Generator().manual_seed(13)
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32).to(DEV)
    wts, gate = torch.rand(T, k, generator=g).to(DEV), torch.rand(T, generator=g).to(DEV)
    n = T * k
    act = ops.gemm(x, gu_all, epilogue=ops.EPI_GATED, pair_ids=ids, pair_div=k, always=(S, T, True))
    y = ops.gemm(act, dn_all, epilogue=ops.EPI_STORE_F32, pair_ids=ids, always=(S, T, False))
    assert act.shape == (n + S * T, I) and y.shape == (n + S * T, H)
    # the routed rows are what the products without the pieces give
    assert torch.equal(act[:n], ops.gemm(x, w_gu, epilogue=ops.EPI_GATED, pair_ids=ids, pair_div=k))
    h = torch.zeros(T, H, device=DEV)
    ops.moe_combine(h, y[:n], None, wts, k, shared=y[n:].view(S, T, H), gate=gate)
    xd = x.double().cpu()
    ref = torch.zeros(T, H, dtype=torch.float64)
    for t in range(T):
        for j in range(k):
            e = int(ids[t, j])
            a = (plain.silu(xd[t] @ w_gu[e, :I].double().cpu().T) * (xd[t] @ w_gu[e, I:].double().cpu().T)).to(dtype).double()
            ref[t] += float(wts[t, j]) * (a @ w_dn[e].double().cpu().T)
        a = (plain.silu(xd[t] @ sg.double().cpu().T) * (xd[t] @ su.double().cpu().T)).to(dtype).double()
        ref[t] += float(gate[t]) * (a @ sd.double().cpu().T)
    close(h, ref, dtype, "routed + gated shared")


@pytest.mark.parametrize("T,E,k,I,H", [(1, 4, 2, 64, 64), (8, 60, 4, 1408, 2048), (40, 6, 3, 128, 192), (300, 8, 2, 64, 128),
                                        (520, 4, 3, 128, 256), (2048, 60, 4, 192, 256)])
def test_weights_in_slabs_of_64_k(T, E, k, I, H):
    """the same products from weights stored [K/64][rows][64]: bit for bit what plain rows give, for
    few rows, many rows, sorted and unsorted pairs, and a plain (not grouped) matrix"""
    from ferrox_amd import ops
    dtype = torch.bfloat16
    x = rnd(T, H, dtype=dtype)
    w_gu, w_dn = rnd(E, 2 * I, H, dtype=dtype, seed=1, scale=0.3), rnd(E, H, I, dtype=dtype, seed=2, scale=0.3)
    kb_gu, kb_dn = ops.to_kblocked(w_gu), ops.to_kblocked(w_dn)
    assert kb_gu.shape == (E, H // 64, 2 * I, 64) and torch.equal(kb_gu[1, 0, 5], w_gu[1, 5, :64])
    g = torch.Generator().manual_seed(17)
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32).to(DEV)
    offsets, sorted_token, sorted_pair, inv = ops.moe_align(ids, E)
    act = ops.gemm(x, w_gu, epilogue=ops.EPI_GATED, a_rows=sorted_token, expert_offsets=offsets, n_rows=T * k)
    act_kb = ops.gemm(x, kb_gu, epilogue=ops.EPI_GATED, a_rows=sorted_token, expert_offsets=offsets, n_rows=T * k,
                      w_kblocked=True)
    assert torch.equal(act, act_kb)
    y = ops.gemm(act, w_dn, epilogue=ops.EPI_STORE_F32, expert_offsets=offsets, c_rows=sorted_pair)
    y_kb = ops.gemm(act, kb_dn, epilogue=ops.EPI_STORE_F32, expert_offsets=offsets, c_rows=sorted_pair, w_kblocked=True)
    assert torch.equal(y, y_kb)
    if T * k <= 64:
        assert torch.equal(ops.gemm(x, kb_gu, epilogue=ops.EPI_GATED, pair_ids=ids, pair_div=k, w_kblocked=True),
                           ops.gemm(x, w_gu, epilogue=ops.EPI_GATED, pair_ids=ids, pair_div=k))
    # a plain matrix with bias, stored, and added into a residual
    bias = rnd(2 * I, dtype=dtype, seed=3)
    assert torch.equal(ops.gemm(x, kb_gu[0], bias=bias, w_kblocked=True), ops.gemm(x, w_gu[0], bias=bias))
    h1, h2 = rnd(T, 2 * I, seed=4), rnd(T, 2 * I, seed=4)
    ops.gemm(x, w_gu[0], epilogue=ops.EPI_RESID, out=h1)
    ops.gemm(x, kb_gu[0], epilogue=ops.EPI_RESID, out=h2, w_kblocked=True)
    assert torch.equal(h1, h2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm_and_embed(dtype):
    from ferrox_amd import ops
    for T, H, eps in [(1, 64, 1e-6), (5, 96, 1e-5), (3, 1000, 1e-3), (2, 4100, 1e-6)]:
        h = rnd(T, H, scale=3.0)
        w = rnd(H, dtype=dtype, seed=1)
        ref = plain.rms_norm(h.double().cpu(), w.double().cpu(), eps)
        close(ops.rmsnorm(h, w, eps, dtype), ref, dtype, f"rmsnorm {T}x{H}")
        rows = torch.tensor([T - 1, 0], dtype=torch.int32, device=DEV)
        close(ops.rmsnorm(h, w, eps, dtype, rows=rows), ref[[T - 1, 0]], dtype, "rmsnorm rows")
    table = rnd(50, 72, dtype=dtype)
    ids = torch.tensor([3, 49, 0, 3], dtype=torch.int32, device=DEV)
    assert torch.equal(ops.embed(table, ids), table[ids.long()].float())


def paged_setup(dtype, nh, nkv, hd, bs, seq_lens, theta, rot, n_pages, seed=0):
    """Random q, k, v for whole sequences; pages filled through rope_kv_write with a shuffled page order."""
    from ferrox_amd import ops
    rng = random.Random(seed)
    free = list(range(n_pages))
    rng.shuffle(free)
    max_blocks = max(-(-L // bs) for L in seq_lens)
    table = torch.zeros(len(seq_lens), max_blocks, dtype=torch.int32)
    toks = []
    for s, L in enumerate(seq_lens):
        for b in range(-(-L // bs)):
            table[s, b] = free.pop()
        toks += [(s, p) for p in range(L)]
    T = len(toks)
    q, k, v = rnd(T, nh * hd, dtype=dtype), rnd(T, nkv * hd, dtype=dtype, seed=1), rnd(T, nkv * hd, dtype=dtype, seed=2)
    # slots that no token is written to hold NaN: nothing may depend on what lies past a sequence's end
    k_pages = torch.full((n_pages, nkv, bs, hd), float("nan"), dtype=dtype, device=DEV)
    v_pages = torch.full((n_pages, nkv, hd, bs), float("nan"), dtype=dtype, device=DEV)
    pos = torch.tensor([p for _, p in toks], dtype=torch.int32, device=DEV)
    seq = torch.tensor([s for s, _ in toks], dtype=torch.int32, device=DEV)
    q_rot = q.clone()
    ops.rope_kv_write(q_rot, k, v, pos, seq, table.to(DEV), k_pages, v_pages, nh, nkv, hd, bs, rot, theta)
    return q, k, v, q_rot, k_pages, v_pages, table.to(DEV), pos, seq, toks


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,hd,bs,rot,theta", [(4, 4, 16, 16, 16, 1e4), (3, 1, 32, 8, 32, 1e6), (6, 3, 48, 4, 24, 5e4),
                                                    (2, 2, 128, 64, 128, 1e6), (8, 2, 80, 16, 80, 1e4)])
def test_rope_and_cache_write(dtype, nh, nkv, hd, bs, rot, theta):
    seq_lens = [5, 2 * bs + 3, 1]
    q, k, v, q_rot, k_pages, v_pages, table, pos, seq, toks = paged_setup(dtype, nh, nkv, hd, bs, seq_lens, theta, rot, 12)
    qd, kd = q.double().cpu().reshape(-1, nh, hd), k.double().cpu().reshape(-1, nkv, hd)
    for t, (s, p) in enumerate(toks):
        want_q = torch.cat([plain.rope_neox(qd[t][:, :rot], p, theta), qd[t][:, rot:]], dim=-1)
        close(q_rot[t].reshape(nh, hd), want_q, dtype, f"q rope token {t}")
        want_k = torch.cat([plain.rope_neox(kd[t][:, :rot], p, theta), kd[t][:, rot:]], dim=-1)
        page = int(table[s, p // bs])
        close(k_pages[page, :, p % bs, :], want_k, dtype, f"k page token {t}")
        assert torch.equal(v_pages[page, :, :, p % bs].reshape(-1), v[t]), f"v page token {t}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,hd,bs,rot,seq_lens", [(4, 2, 128, 64, 128, [300, 7, 330]), (3, 1, 80, 64, 48, [640, 5]),
                                                       (2, 2, 64, 16, 64, [530, 40]), (2, 1, 96, 128, 96, [520])])
def test_rope_and_cache_write_of_long_prompts(dtype, nh, nkv, hd, bs, rot, seq_lens):
    """Many tokens, eight pairs to a thread: pages that begin or end inside a sequence, page sizes other than 64,
    tokens of another sequence between."""
    theta = 1e6
    n_pages = sum(-(-L // bs) for L in seq_lens) + 2
    q, k, v, q_rot, k_pages, v_pages, table, pos, seq, toks = paged_setup(dtype, nh, nkv, hd, bs, seq_lens, theta, rot, n_pages)
    assert len(toks) >= 512
    T = len(toks)
    p = pos.double().cpu()
    freq = 1.0 / theta ** (torch.arange(0, rot, 2, dtype=torch.float64) / rot)
    # plain.rope_neox(..., "float32"), all tokens at once: the float32 product of position and float32 frequency
    ang = (p.float()[:, None] * freq.float()[None, :]).double()
    def rotated(x, heads):
        x = x.double().cpu().reshape(T, heads, hd)
        a, b = x[..., :rot // 2], x[..., rot // 2:rot]
        c, s_ = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
        return torch.cat([a * c - b * s_, a * s_ + b * c, x[..., rot:]], dim=-1)
    for t in (5, T - 1):
        assert torch.allclose(plain.rope_neox(q[t].double().cpu().reshape(nh, hd)[:, :rot], int(pos[t]), theta, "float32"),
                              rotated(q, nh)[t, :, :rot], atol=1e-12)  # the formula above is the plain one
    near = lambda got, want, what: close(got, want, dtype, what)
    near(q_rot.reshape(T, nh, hd), rotated(q, nh), "rotated queries")
    page_of = table.cpu()[seq.cpu().long(), (pos.cpu() // bs).long()].long()
    slot = (pos.cpu() % bs).long()
    near(k_pages.cpu()[page_of, :, slot, :], rotated(k, nkv), "key pages")
    assert torch.equal(v_pages.cpu()[page_of, :, :, slot], v.cpu().reshape(T, nkv, hd)), "value pages"
    used = torch.zeros(n_pages, bs, dtype=torch.bool)
    used[page_of, slot] = True
    assert bool(torch.isnan(v_pages.cpu().float().permute(0, 3, 1, 2)[~used]).all()), "slots past the sequences stay untouched"


DEEP_POSITIONS = [0, 1, 511, 2047, 2048, 4097, 8191, 16384, 20000, 32766, 32767]


def rotated_by_float32_angles(x, positions, rot, theta, angles="float32"):
    """x [T, heads, hd] in float64 with its first `rot` dimensions turned, split halves, by the plain model's angles"""
    out = x.clone()
    for t, p in enumerate(positions):
        out[t, :, :rot] = plain.rope_neox(x[t, :, :rot], int(p), theta, angles)
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,hd,bs,rot,theta", [(2, 1, 128, 64, 128, 1e6), (3, 3, 64, 16, 32, 1e4), (2, 2, 16, 16, 16, 1e6)])
def test_rope_deep_in_a_sequence(dtype, nh, nkv, hd, bs, rot, theta):
    """Rotation and cache write at positions up to 32,767.  The angle is the float32 product of the position and
    the float32 frequency (ferrox-core/src/attention.rs:26-27); against float64 sines and cosines of exactly that
    angle the float32 kernel is right to rounding, and would be off by a thousand times that against exact angles."""
    from ferrox_amd import ops
    T = len(DEEP_POSITIONS)
    blocks = -(-32768 // bs)
    table = torch.zeros(1, blocks, dtype=torch.int32)
    used = sorted({p // bs for p in DEEP_POSITIONS})
    order = torch.randperm(len(used), generator=torch.Generator().manual_seed(bs)).tolist()
    for b, page in zip(used, order):
        table[0, b] = page + 1                             # page 0 stays empty
    q, k, v = rnd(T, nh * hd, dtype=dtype), rnd(T, nkv * hd, dtype=dtype, seed=1), rnd(T, nkv * hd, dtype=dtype, seed=2)
    k_pages = torch.full((len(used) + 1, nkv, bs, hd), float("nan"), dtype=dtype, device=DEV)
    v_pages = torch.full((len(used) + 1, nkv, hd, bs), float("nan"), dtype=dtype, device=DEV)
    pos = torch.tensor(DEEP_POSITIONS, dtype=torch.int32, device=DEV)
    seq = torch.zeros(T, dtype=torch.int32, device=DEV)
    q_rot = q.clone()
    ops.rope_kv_write(q_rot, k, v, pos, seq, table.to(DEV), k_pages, v_pages, nh, nkv, hd, bs, rot, theta)
    want_q = rotated_by_float32_angles(q.double().cpu().reshape(T, nh, hd), DEEP_POSITIONS, rot, theta)
    want_k = rotated_by_float32_angles(k.double().cpu().reshape(T, nkv, hd), DEEP_POSITIONS, rot, theta)
    page_of = table[0, (pos.cpu() // bs).long()].long()
    slot = (pos.cpu() % bs).long()
    got_q, got_k = q_rot.reshape(T, nh, hd), k_pages.cpu()[page_of, :, slot, :]
    close(got_q, want_q, dtype, "rotated queries")
    close(got_k, want_k, dtype, "key pages")
    assert torch.equal(v_pages.cpu()[page_of, :, :, slot], v.cpu().reshape(T, nkv, hd)), "value pages"
    assert bool(torch.isnan(k_pages[0].float()).all()), "a page that no position maps to was written"
    if dtype == torch.float32:
        exact = rotated_by_float32_angles(q.double().cpu().reshape(T, nh, hd), DEEP_POSITIONS, rot, theta, "exact")
        off = float((got_q.double().cpu() - exact).abs().max()) / float(exact.abs().max())
        assert off > 1e-4, f"exact angles are only {off:.2e} away: the test does not tell the two apart"


def test_qkv_product_that_rotates_deep_in_a_sequence():
    """the rotating product's epilogue at positions up to 32,767: the bits of the product followed by rope_kv_write,
    which the test above holds against the plain rotation"""
    from ferrox_amd import ops
    T, H, nh, nkv, hd, bs, rot, theta = len(DEEP_POSITIONS), 264, 4, 2, 64, 64, 64, 1e6
    N = (nh + 2 * nkv) * hd
    w = rnd(N, H, dtype=torch.bfloat16, seed=1, scale=0.05)
    b = rnd(N, dtype=torch.bfloat16, seed=2)
    x = rnd(T, H, dtype=torch.bfloat16, seed=3)
    blocks = 32768 // bs
    used = sorted({p // bs for p in DEEP_POSITIONS})
    table = torch.zeros(1, blocks, dtype=torch.int32)
    for i, blk in enumerate(used):
        table[0, blk] = len(used) - i
    table = table.to(DEV)
    pos = torch.tensor(DEEP_POSITIONS, dtype=torch.int32, device=DEV)
    seq = torch.zeros(T, dtype=torch.int32, device=DEV)
    pages = lambda: (torch.zeros(len(used) + 1, nkv, bs, hd, dtype=torch.bfloat16, device=DEV),
                     torch.zeros(len(used) + 1, nkv, hd, bs, dtype=torch.bfloat16, device=DEV))
    assert ops.can_qkv_rope(x, w, T, hd, rot, False)
    k1, v1 = pages()
    got = ops.qkv_rope(x, w, b, pos, seq, table, k1, v1, nh, nkv, hd, bs, rot, theta)
    k2, v2 = pages()
    ref = ops.gemm(x, w, bias=b)
    qw, kvw = nh * hd, nkv * hd
    ops.rope_kv_write(ref[:, :qw], ref[:, qw:qw + kvw], ref[:, qw + kvw:], pos, seq, table, k2, v2, nh, nkv, hd, bs, rot, theta)
    assert torch.equal(got[:, :qw], ref[:, :qw]), "rotated queries"
    assert torch.equal(k1, k2) and float(k1.abs().sum()) > 0, "key pages"
    assert torch.equal(v1, v2), "value pages"


@pytest.mark.parametrize("later", [False, True])
@pytest.mark.parametrize("T,H,nh,nkv,hd,bs,rot,bias", [(1, 2048, 16, 16, 128, 64, 128, True), (8, 2048, 16, 16, 128, 64, 128, True),
                                                       (16, 264, 6, 2, 64, 16, 32, True), (5, 520, 3, 1, 32, 8, 0, False),
                                                       (7, 128, 4, 2, 96, 32, 64, True), (30, 264, 6, 2, 64, 16, 64, True),
                                                       (64, 2048, 16, 16, 128, 64, 128, True), (50, 128, 4, 2, 96, 32, 64, False)])
def test_qkv_product_that_rotates_and_writes_the_cache(later, T, H, nh, nkv, hd, bs, rot, bias):
    """The q/k/v product with rotation and cache write in its epilogue gives the bits of the product followed
    by rope_kv_write: rotated queries, key pages and value pages; also from rows whose norm's scale is applied
    by the product."""
    from ferrox_amd import ops
    N = (nh + 2 * nkv) * hd
    w = rnd(N, H, dtype=torch.bfloat16, seed=1, scale=0.05)
    b = rnd(N, dtype=torch.bfloat16, seed=2) if bias else None
    x = rnd(T, H, dtype=torch.bfloat16, seed=3)
    if later:
        ss = (torch.rand(T, (H + 255) // 256, generator=torch.Generator().manual_seed(4)) * 40 + 1).to(DEV)
        x = ops.ScaleLater(x, ss, 1e-6)
    g = torch.Generator().manual_seed(5)
    n_seq = 3
    seq = torch.randint(0, n_seq, (T,), generator=g)
    pos = torch.zeros(T, dtype=torch.long)
    for s_ in range(n_seq):                       # distinct positions inside a sequence
        idx = (seq == s_).nonzero().flatten()
        pos[idx] = torch.randperm(5 * bs, generator=g)[:idx.numel()]
    table = torch.randperm(n_seq * 5, generator=g).reshape(n_seq, 5).to(torch.int32).to(DEV)
    pos_d, seq_d = pos.to(torch.int32).to(DEV), seq.to(torch.int32).to(DEV)
    pages = lambda: (torch.zeros(n_seq * 5, nkv, bs, hd, dtype=torch.bfloat16, device=DEV),
                     torch.zeros(n_seq * 5, nkv, hd, bs, dtype=torch.bfloat16, device=DEV))
    assert ops.can_qkv_rope(x, w, T, hd, rot, False)
    k1, v1 = pages()
    got = ops.qkv_rope(x, w, b, pos_d, seq_d, table, k1, v1, nh, nkv, hd, bs, rot, 1e6)
    k2, v2 = pages()
    ref = ops.gemm(x.x, w, bias=b, row_ss=(x.ss, x.eps)) if later else ops.gemm(x, w, bias=b)
    qw, kvw = nh * hd, nkv * hd
    ops.rope_kv_write(ref[:, :qw], ref[:, qw:qw + kvw], ref[:, qw + kvw:], pos_d, seq_d, table, k2, v2, nh, nkv, hd, bs, rot, 1e6)
    assert torch.equal(got[:, :qw], ref[:, :qw]), "rotated queries"
    assert torch.equal(k1, k2), "key pages"
    assert torch.equal(v1, v2), "value pages"
    got2 = ops.qkv_rope(x, w, b, pos_d, seq_d, table, None, None, nh, nkv, hd, bs, rot, 1e6)     # no pages: queries only
    assert torch.equal(got2[:, :qw], ref[:, :qw])
    assert not ops.can_qkv_rope(x, w, 65, hd, rot, False) and not ops.can_qkv_rope(x, w, T, hd, rot, True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,hd,bs,rot,interleaved", [(3, 1, 32, 8, 32, False), (2, 2, 64, 16, 32, False),
                                                          (2, 1, 48, 8, 24, True), (4, 2, 128, 64, 128, False)])
def test_rope_with_frequency_factors(dtype, nh, nkv, hd, bs, rot, interleaved):
    """A table of per-pair factors divides the angles (ferrox-core/src/attention.rs:319-333): the rotating
    kernel, and for bfloat16 split halves also the q/k/v product that rotates in its epilogue, against the
    formula; a table of ones gives the bits of no table."""
    from ferrox_amd import ops
    theta, T = 1e4, 20
    g = torch.Generator().manual_seed(rot)
    factors = (1.0 + 7.0 * torch.rand(rot // 2, generator=g)).to(DEV)
    q, k, v = rnd(T, nh * hd, dtype=dtype), rnd(T, nkv * hd, dtype=dtype, seed=1), rnd(T, nkv * hd, dtype=dtype, seed=2)
    pos = torch.arange(3, 3 + T, dtype=torch.int32, device=DEV)
    seq = torch.zeros(T, dtype=torch.int32, device=DEV)
    n_blocks = -(-(3 + T) // bs)
    table = torch.arange(n_blocks, dtype=torch.int32, device=DEV).flip(0)[None].contiguous()
    pages = lambda: (torch.zeros(n_blocks, nkv, bs, hd, dtype=dtype, device=DEV), torch.zeros(n_blocks, nkv, hd, bs, dtype=dtype, device=DEV))

    def want(x, heads):
        x = x.double().cpu().reshape(T, heads, hd)
        i = torch.arange(rot // 2, dtype=torch.float64)
        ang = pos.double().cpu()[:, None] * (1.0 / theta ** (2 * i / rot))[None, :] / factors.double().cpu()[None, :]
        c, s_ = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
        out = x.clone()
        ia, ib = (2 * i.long(), 2 * i.long() + 1) if interleaved else (i.long(), i.long() + rot // 2)
        out[..., ia], out[..., ib] = x[..., ia] * c - x[..., ib] * s_, x[..., ia] * s_ + x[..., ib] * c
        return out

    kp, vp = pages()
    q1 = q.clone()
    ops.rope_kv_write(q1, k, v, pos, seq, table, kp, vp, nh, nkv, hd, bs, rot, theta, interleaved, freq_factors=factors)
    close(q1.reshape(T, nh, hd), want(q, nh), dtype, "rotated queries")
    page_of, slot = table[0].cpu()[(pos.cpu() // bs).long()].long(), (pos.cpu() % bs).long()
    close(kp.cpu()[page_of, :, slot, :], want(k, nkv), dtype, "key pages")
    # a table of ones is no table
    ones = torch.ones(rot // 2, device=DEV)
    kp1, vp1 = pages()
    kp0, vp0 = pages()
    qa, qb = q.clone(), q.clone()
    ops.rope_kv_write(qa, k, v, pos, seq, table, kp1, vp1, nh, nkv, hd, bs, rot, theta, interleaved, freq_factors=ones)
    ops.rope_kv_write(qb, k, v, pos, seq, table, kp0, vp0, nh, nkv, hd, bs, rot, theta, interleaved)
    assert torch.equal(qa, qb) and torch.equal(kp1, kp0)
    with pytest.raises(ops.KernelError):
        ops.rope_kv_write(qa, k, v, pos, seq, table, kp1, vp1, nh, nkv, hd, bs, rot, theta, interleaved, freq_factors=ones[:-1])
    if dtype == torch.bfloat16 and not interleaved and rot % 32 == 0 and hd % 32 == 0:
        H = 96
        w = rnd((nh + 2 * nkv) * hd, H, dtype=dtype, seed=5, scale=0.1)
        x = rnd(T, H, dtype=dtype, seed=6)
        assert ops.can_qkv_rope(x, w, T, hd, rot, False)
        k1, v1 = pages()
        got = ops.qkv_rope(x, w, None, pos, seq, table, k1, v1, nh, nkv, hd, bs, rot, theta, freq_factors=factors)
        ref = ops.gemm(x, w)
        qw, kvw = nh * hd, nkv * hd
        k2, v2 = pages()
        ops.rope_kv_write(ref[:, :qw], ref[:, qw:qw + kvw], ref[:, qw + kvw:], pos, seq, table, k2, v2, nh, nkv, hd, bs, rot,
                          theta, freq_factors=factors)
        assert torch.equal(got[:, :qw], ref[:, :qw]) and torch.equal(k1, k2) and torch.equal(v1, v2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,hd,bs,window", [(4, 4, 16, 16, 0), (3, 1, 32, 8, 16), (6, 3, 48, 4, 40), (2, 2, 128, 64, 0),
                                                 (8, 2, 80, 16, 7), (4, 1, 256, 32, 100), (4, 2, 64, 64, 50), (3, 1, 128, 128, 90),
                                                 (2, 1, 64, 64, 0), (2, 2, 128, 64, 70)])
def test_attention_kernels(dtype, nh, nkv, hd, bs, window):
    """Whole sequences through the tiled kernel, and their last tokens again through the decode
    kernel, against the plain attention on the same rotated, rounded q/k/v."""
    from ferrox_amd import ops
    seq_lens = [70, 1, 33, 150]
    theta = 1e4
    q, k, v, q_rot, k_pages, v_pages, table, pos, seq, toks = paged_setup(dtype, nh, nkv, hd, bs, seq_lens, theta, hd, 128)
    T = len(toks)
    scale = 1.0 / math.sqrt(hd)
    # reference from what the pages hold
    ref = torch.zeros(T, nh, hd, dtype=torch.float64)
    starts = [0]
    for L in seq_lens:
        starts.append(starts[-1] + L)
    kp, vp, tab = k_pages.double().cpu(), v_pages.double().cpu(), table.cpu()
    for s, L in enumerate(seq_lens):
        ks = torch.stack([kp[int(tab[s, p // bs]), :, p % bs, :] for p in range(L)])
        vs = torch.stack([vp[int(tab[s, p // bs]), :, :, p % bs] for p in range(L)])
        qs = q_rot[starts[s]:starts[s + 1]].double().cpu().reshape(L, nh, hd)
        ref[starts[s]:starts[s + 1]] = plain.causal_attention(qs, ks, vs, nh, nkv, window or None)
    ref = ref.reshape(T, nh * hd)
    # blocks of up to 64 queries
    t_seq, t_tok, t_n = [], [], []
    for s, L in enumerate(seq_lens):
        for t0 in range(0, L, 64):
            t_seq.append(s); t_tok.append(starts[s] + t0); t_n.append(min(64, L - t0))
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    from ferrox_amd import debug
    for groups in (1, 2):      # of waves per block of the kernel for pages of 64 keys (it takes two where blocks are few)
        out = torch.zeros(T, nh * hd, dtype=dtype, device=DEV)
        with debug.kernel_switch("attention", "direct_groups", groups):
            ops.attention_tiles(q_rot, out, k_pages, v_pages, table, pos, i32(t_seq), i32(t_tok), i32(t_n), nh, nkv, hd, bs, window, scale)
        close(out, ref, dtype, f"tiled attention, {groups} group(s) of waves")
    tq = ops.attention_tile_queries(dtype, hd, bs)
    assert tq == (128 if dtype == torch.bfloat16 and bs % 64 == 0 and hd in (64, 128) else 64)
    if tq > 64:       # larger items where the kernel takes them: blocks of eight waves
        t_seq, t_tok, t_n = [], [], []
        for s, L in enumerate(seq_lens):
            for t0 in range(0, L, tq):
                t_seq.append(s); t_tok.append(starts[s] + t0); t_n.append(min(tq, L - t0))
        for groups in (1, 2):
            wide = torch.zeros(T, nh * hd, dtype=dtype, device=DEV)
            with debug.kernel_switch("attention", "direct_groups", groups):
                ops.attention_tiles(q_rot, wide, k_pages, v_pages, table, pos, i32(t_seq), i32(t_tok), i32(t_n), nh, nkv, hd, bs, window,
                                    scale, tile_q=tq)
            close(wide, ref, dtype, f"tiled attention, items of {tq}, {groups} group(s) of waves")
    else:
        with pytest.raises(ops.KernelError):
            ops.attention_tiles(q_rot, out, k_pages, v_pages, table, pos, i32(t_seq), i32(t_tok), i32(t_n), nh, nkv, hd, bs, window,
                                scale, tile_q=128)
    # the last token of every sequence as a single query
    out2 = torch.zeros(T, nh * hd, dtype=dtype, device=DEV)
    last = [starts[s + 1] - 1 for s in range(len(seq_lens))]
    for chunk in (64, 256):
        ops.attention_decode(q_rot, out2, k_pages, v_pages, table, pos, i32(list(range(len(seq_lens)))), i32(last),
                             nh, nkv, hd, bs, window, scale, max_kv_len=max(seq_lens), chunk=chunk)
        close(out2[last], ref[last], dtype, f"decode attention chunk {chunk}")


@pytest.mark.parametrize("hd,bs,window", [(64, 16, 0), (64, 64, 0), (128, 64, 40000), (32, 16, 9000)])
def test_attention_over_more_pages_than_a_block_copies(hd, bs, window):
    """A sequence of more than 1024 pages (the kernels copy that many page ids into LDS and read the rest of
    the table from memory): its last 64 tokens as a block of queries, and its last token alone."""
    from ferrox_amd import ops
    nh, nkv, dtype = 2, 1, torch.bfloat16
    L = bs * 1030 + 5
    q, k, v, q_rot, k_pages, v_pages, table, pos, seq, toks = paged_setup(dtype, nh, nkv, hd, bs, [L], 1e6, hd, 1040)
    scale = 1.0 / math.sqrt(hd)
    kp, vp, tab = k_pages.double().cpu(), v_pages.double().cpu(), table.cpu()[0].long()
    ks = kp[tab].permute(0, 2, 1, 3).reshape(-1, nkv, hd)[:L]                  # [L, nkv, hd]
    vs = vp[tab].permute(0, 3, 1, 2).reshape(-1, nkv, hd)[:L]
    qs = q_rot[L - 64:].double().cpu().reshape(64, nh, hd)
    ref = torch.zeros(64, nh, hd, dtype=torch.float64)
    for i in range(64):
        p = L - 64 + i
        lo = max(0, p - window + 1) if window else 0
        for h in range(nh):
            sc = (ks[lo:p + 1, 0] @ qs[i, h]) * scale
            ref[i, h] = torch.softmax(sc, 0) @ vs[lo:p + 1, 0]
    ref = ref.reshape(64, nh * hd)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    out = torch.zeros(L, nh * hd, dtype=dtype, device=DEV)
    ops.attention_tiles(q_rot, out, k_pages, v_pages, table, pos, i32([0]), i32([L - 64]), i32([64]), nh, nkv, hd, bs, window, scale)
    close(out[L - 64:], ref, dtype, "tiled attention, last block")
    out2 = torch.zeros(L, nh * hd, dtype=dtype, device=DEV)
    for chunk in (None, 4096):
        ops.attention_decode(q_rot, out2, k_pages, v_pages, table, pos, i32([0]), i32([L - 1]), nh, nkv, hd, bs, window, scale,
                             max_kv_len=L, chunk=chunk)
        close(out2[L - 1], ref[63], dtype, f"decode attention chunk {chunk}")


def test_decode_attention_of_a_short_sequence_beside_a_very_long_one():
    """One launch, no window, two chunks: a sequence of 2,500 pages, whose chunks span more pages than a block
    copies into LDS (1024), beside one of 300 keys.  The short sequence's chunks lie far below the range of page
    ids that its blocks copy (the range is laid out for the launch's longest chunk before the position is known),
    so every one of its lookups goes to the table in memory; both against the plain attention."""
    from ferrox_amd import ops
    nh, nkv, hd, bs, dtype = 4, 2, 64, 16, torch.bfloat16
    lens = [40005, 300]
    n_pages = sum(-(-L // bs) for L in lens) + 3
    q, k, v, q_rot, k_pages, v_pages, table, pos, seq, toks = paged_setup(dtype, nh, nkv, hd, bs, lens, 1e6, hd, n_pages)
    scale = 1.0 / math.sqrt(hd)
    kp, vp = k_pages.double().cpu(), v_pages.double().cpu()
    last = [lens[0] - 1, lens[0] + lens[1] - 1]                               # token numbers of the two last positions
    out = torch.zeros(len(toks), nh * hd, dtype=dtype, device=DEV)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    chunk = 20032                                                             # 1,252 pages a chunk
    assert chunk // bs > 1024
    ops.attention_decode(q_rot, out, k_pages, v_pages, table, pos, i32([0, 1]), i32(last), nh, nkv, hd, bs, 0, scale,
                         max_kv_len=lens[0], chunk=chunk)
    for s_, L in enumerate(lens):
        tab = table.cpu()[s_].long()[: -(-L // bs)]
        ks = kp[tab].permute(0, 2, 1, 3).reshape(-1, nkv, hd)[:L]
        vs = vp[tab].permute(0, 3, 1, 2).reshape(-1, nkv, hd)[:L]
        qs = q_rot[last[s_]].double().cpu().reshape(nh, hd)
        ref = torch.stack([torch.softmax((ks[:, h // (nh // nkv)] @ qs[h]) * scale, 0) @ vs[:, h // (nh // nkv)] for h in range(nh)])
        close(out[last[s_]].reshape(nh, hd), ref, dtype, f"sequence of {L} keys")


def test_decode_attention_of_more_sequences_than_fill_the_cus_once():
    """20 sequences of 16 kv heads are 320 blocks for 256 CUs: the chunks are then chosen by how full the blocks' last
    round would be (eight a sequence here, one with 16 sequences), and sequences of every length, down to one key and
    up to the bound, must come out as plain attention gives them, with the chunks chosen and with one."""
    from ferrox_amd import ops
    nh, nkv, hd, bs, dtype = 16, 16, 64, 64, torch.bfloat16
    lens = [1100, 1, 64, 65, 1087, 1088, 1089, 700, 513, 128] * 2
    n_pages = sum(-(-L // bs) for L in lens) + 3
    q, k, v, q_rot, k_pages, v_pages, table, pos, seq, toks = paged_setup(dtype, nh, nkv, hd, bs, lens, 1e6, hd, n_pages)
    scale = 1.0 / math.sqrt(hd)
    kp, vp = k_pages.double().cpu(), v_pages.double().cpu()
    ends, last = 0, []
    for L in lens:
        ends += L
        last.append(ends - 1)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    outs = []
    for chunk in (None, 1152):
        out = torch.zeros(len(toks), nh * hd, dtype=dtype, device=DEV)
        ops.attention_decode(q_rot, out, k_pages, v_pages, table, pos, i32(list(range(len(lens)))), i32(last), nh, nkv, hd, bs, 0,
                             scale, max_kv_len=1152, chunk=chunk)
        outs.append(out)
    for s_, L in enumerate(lens):
        tab = table.cpu()[s_].long()[: -(-L // bs)]
        ks = kp[tab].permute(0, 2, 1, 3).reshape(-1, nkv, hd)[:L]
        vs = vp[tab].permute(0, 3, 1, 2).reshape(-1, nkv, hd)[:L]
        qs = q_rot[last[s_]].double().cpu().reshape(nh, hd)
        ref = torch.stack([torch.softmax((ks[:, h] @ qs[h]) * scale, 0) @ vs[:, h] for h in range(nh)])
        for out, what in zip(outs, ("chunks as chosen", "one chunk")):
            close(out[last[s_]].reshape(nh, hd), ref, dtype, f"sequence {s_} of {L} keys, {what}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,H,E,k,renorm", [(1, 64, 8, 2, False), (7, 96, 6, 3, True), (33, 200, 60, 4, False),
                                             (5, 128, 130, 8, True), (4, 72, 5, 5, False)])
def test_router(dtype, T, H, E, k, renorm):
    """router matrix product + selection, with the shared expert's gate as an extra row"""
    from ferrox_amd import ops
    x, wr, sg = rnd(T, H, dtype=dtype), rnd(E, H, dtype=dtype, seed=1, scale=0.3), rnd(H, dtype=dtype, seed=2, scale=0.2)
    logits = ops.gemm(x, torch.cat([wr, sg[None]]).contiguous(), epilogue=ops.EPI_STORE_F32)
    ids, w, gate = ops.router_select(logits, E, k, renorm, has_gate=True)
    xd, wd = x.double().cpu(), wr.double().cpu()
    for t in range(T):
        want_ids, want_w = plain.route_top_k(wd @ xd[t], k, renorm)
        assert ids[t].tolist() == want_ids, f"token {t}: experts {ids[t].tolist()} != {want_ids}"
        close(w[t], want_w, torch.float32, f"router weights token {t}")
    close(gate, torch.sigmoid(xd @ sg.double().cpu()), torch.float32, "shared gate")
    # the product the other way round (router rows as the short side), read through its transpose
    logits_t = ops.gemm(torch.cat([wr, sg[None]]).contiguous(), x, epilogue=ops.EPI_STORE_F32).t()
    assert logits_t.shape == logits.shape and logits_t.stride(1) != 1 or T == 1
    ids_t, w_t, gate_t = ops.router_select(logits_t, E, k, renorm, has_gate=True)
    assert torch.equal(ids_t, ids)
    close(w_t, w, torch.float32, "router weights from transposed logits")
    close(gate_t, gate, torch.float32, "shared gate from transposed logits")


def test_router_golden_vector():
    """logits 1..8, k=3, no renormalisation -> experts [7, 6, 5], weights [0.6323223, 0.2326232,
    0.0855683] (the vector of the reference's own test, ferrox-moe/src/lib.rs:863-893)."""
    from ferrox_amd import ops
    logits = torch.arange(1, 9, dtype=torch.float32, device=DEV)[None].contiguous()
    ids, w, _ = ops.router_select(logits, 8, 3, False)
    assert ids[0].tolist() == [7, 6, 5]
    assert torch.allclose(w[0].cpu(), torch.tensor([0.6323223, 0.2326232, 0.0855683]), atol=1e-4)   # its tolerance
    assert abs(float(w[0].sum()) - 0.9505138) < 1e-4
    exact = torch.softmax(torch.arange(1, 9, dtype=torch.float64), 0).flip(0)[:3]
    assert torch.allclose(w[0].cpu().double(), exact, atol=1e-6)
    ids, w, _ = ops.router_select(logits, 8, 3, True)              # renormalised: the same experts, sum 1
    assert ids[0].tolist() == [7, 6, 5] and abs(float(w[0].sum()) - 1.0) < 1e-6
    ids, w, _ = ops.router_select(torch.zeros(1, 8, device=DEV), 8, 3, True)     # all equal: lowest indices
    assert ids[0].tolist() == [0, 1, 2] and torch.allclose(w[0].cpu(), torch.full((3,), 1 / 3))
    ids, w, _ = ops.router_select(torch.tensor([[0.1, 5.0, 0.2, 3.0, -1.0]], device=DEV), 5, 2, False)
    assert ids[0].tolist() == [1, 3]                               # ferrox-moe/src/lib.rs:834-841


# xorshift64 started from a small number returns small numbers at first (the first uniform draw is 0, which picks
# the first token that has any probability whatever the logits say); the sampling tests start it high
SEED = 0x2545F4914F6CDD1D


def test_sampling_kernel():
    from ferrox_amd import ops
    V = 1000
    logits = rnd(6, V, scale=3.0)
    assert ops.sample(logits).tolist() == logits.argmax(-1).tolist()
    tie = torch.zeros(1, V, device=DEV)
    tie[0, [17, 400]] = 5.0
    assert ops.sample(tie).tolist() == [17]
    # seeded sampling against the plain sampler, option by option
    cases = [dict(temperature=0.8), dict(temperature=1.3, top_k=5), dict(temperature=0.7, top_p=0.6),
             dict(temperature=1.0, top_k=50, top_p=0.9, repetition_penalty=1.3),
             dict(temperature=0.0, repetition_penalty=2.0, presence_penalty=0.5, frequency_penalty=0.25),
             dict(temperature=0.9, top_k=1)]
    hist = [int(logits[0].argmax()), 3, 3, 999, int(logits[0].argmax())]
    draws = []
    for case in cases:
        picked = set()
        for trial in range(12):
            seed = SEED + (trial << 45)
            want = plain.sample(logits[0].double().cpu().tolist(), plain.XorShift64(seed), history=hist, **case)
            u = plain.XorShift64(seed).next_f32()
            draws.append(u)
            f = lambda v: torch.tensor([v], dtype=torch.float32, device=DEV)
            got = ops.sample(logits[:1], temperature=f(case.get("temperature", 0.0)), draw=f(u),
                             top_k=torch.tensor([case.get("top_k", 0)], dtype=torch.int32, device=DEV),
                             top_p=f(case.get("top_p", 1.0)), rep_penalty=f(case.get("repetition_penalty", 1.0)),
                             presence=f(case.get("presence_penalty", 0.0)), frequency=f(case.get("frequency_penalty", 0.0)),
                             hist=torch.tensor(hist, dtype=torch.int32, device=DEV),
                             hist_start=torch.tensor([0, len(hist)], dtype=torch.int32, device=DEV)).tolist()[0]
            assert got == want, f"{case} trial {trial}: kernel {got}, plain {want}"
            picked.add(got)
        if case["temperature"] > 0 and case.get("top_k", 0) != 1:
            assert len(picked) >= 3, f"{case}: twelve draws picked {sorted(picked)} only"
    assert min(draws) > 0.0 and max(draws) - min(draws) > 0.5, "the draws do not spread over (0, 1)"


def test_sampling_kernel_at_the_real_vocabulary():
    """V = 151,936, three rows in one call, eight draws each: the command line's defaults (top-k 40, top-p 0.95,
    repetition penalty 1.1: ferrox-cli/src/run.rs:52-64) and temperature alone, against the plain sampler
    (ferrox-models/src/sampling.rs:93-189).  A few dozen tokens stand out of the noise, as in a trained model, so
    that the most likely token has a probability near 0.2 and top-p cuts inside the top-k."""
    from ferrox_amd import ops
    V, R = 151936, 3
    g = torch.Generator().manual_seed(11)
    logits = torch.randn(R, V, generator=g) * 2.0
    for r in range(R):
        idx = torch.randperm(V, generator=g)[:30]
        logits[r, idx] += 5.0 + 3.0 * torch.rand(30, generator=g)
    rows = logits.double().tolist()
    dev = logits.to(DEV)
    assert ops.sample(dev).tolist() == logits.argmax(-1).tolist()
    hists = [[int(logits[0].argmax()), 7, 7, V - 1], [], [int(logits[2].argmax())] * 3 + [int(logits[2].topk(2).indices[1])]]
    flat = [t for h in hists for t in h]
    starts = [0]
    for h in hists:
        starts.append(starts[-1] + len(h))
    f = lambda v: torch.tensor(v, dtype=torch.float32, device=DEV)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    for case in (dict(temperature=0.8, top_k=40, top_p=0.95, repetition_penalty=1.1), dict(temperature=0.8)):
        gens = [plain.XorShift64(SEED + ((r + 1) << 45)) for r in range(R)]
        mirrors = [plain.XorShift64(SEED + ((r + 1) << 45)) for r in range(R)]
        picked = [set() for _ in range(R)]
        for draw in range(8):
            want = [plain.sample(rows[r], gens[r], history=hists[r], **case) for r in range(R)]
            u = [m.next_f32() for m in mirrors]
            got = ops.sample(dev, temperature=f([case["temperature"]] * R), draw=f(u), top_k=i32([case.get("top_k", 0)] * R),
                             top_p=f([case.get("top_p", 1.0)] * R), rep_penalty=f([case.get("repetition_penalty", 1.0)] * R),
                             presence=f([0.0] * R), frequency=f([0.0] * R), hist=i32(flat), hist_start=i32(starts)).tolist()
            assert got == want, f"{case} draw {draw}: kernel {got}, plain {want}"
            for r in range(R):
                picked[r].add(got[r])
        assert all(len(p) >= 3 for p in picked), f"{case}: eight draws picked {picked}"


@pytest.mark.parametrize("M,N,K", [(1, 6144, 2048), (8, 6144, 2048), (5, 100, 96), (16, 48, 264), (31, 257, 520),
                                    (32, 2560, 1792)])
@pytest.mark.parametrize("gamma_dtype", [torch.bfloat16, torch.float32])
def test_gemm_with_fused_norm(M, N, K, gamma_dtype):
    """RMSNorm applied inside the product against norm kernel + product and against the plain norm"""
    from ferrox_amd import ops
    h = rnd(M, K, scale=2.0)
    gamma = (1.0 + rnd(K, seed=3, scale=0.2)).to(gamma_dtype)
    w, bias = rnd(N, K, dtype=torch.bfloat16, seed=1, scale=0.05), rnd(N, dtype=torch.bfloat16, seed=2)
    eps = 1e-6
    assert ops.can_fuse_norm(h, w, M)
    got = ops.gemm(h, w, bias=bias, norm=(gamma, eps))
    two = ops.gemm(ops.rmsnorm(h, gamma, eps, torch.bfloat16), w, bias=bias)
    want = plain.rms_norm(h.double().cpu(), gamma.double().cpu(), eps) @ w.double().cpu().T + bias.double().cpu()
    close(got, want, torch.bfloat16, "fused norm product")
    close(two, want, torch.bfloat16, "norm, then product")
    assert not ops.can_fuse_norm(rnd(33, K), w, 33)


@pytest.mark.parametrize("T,H,E,k,renorm,has_gate", [(1, 2048, 60, 4, False, True), (8, 2048, 60, 4, False, True),
                                                      (16, 264, 7, 3, True, False), (5, 1792, 130, 8, True, True), (16, 2048, 60, 4, False, True),
                                                      (64, 2048, 60, 4, False, True), (33, 96, 6, 3, True, True),
                                                      (3, 64, 4, 4, False, True), (130, 1792, 60, 4, False, True),
                                                      (256, 264, 64, 8, True, True)])
def test_moe_front(T, H, E, k, renorm, has_gate):
    """norm + router products + selection + sort in one launch, twice in a row (the kernel's counter
    must be back at zero), against the plain norm and router on the rounded activations"""
    from ferrox_amd import ops
    h = rnd(T + 2, H, scale=1.5)[1:T + 1]                                    # a view that starts past row 0
    gamma = (1.0 + rnd(H, seed=3, scale=0.2)).to(torch.bfloat16)
    router = rnd(E + (1 if has_gate else 0), H, dtype=torch.bfloat16, seed=4, scale=0.3)
    eps = 1e-5
    x_sep = ops.rmsnorm(h.contiguous(), gamma, eps, torch.bfloat16)
    for rep in range(3):
        # the third time with the sort by expert in the same launch, and two pieces behind the experts
        got = ops.moe_front(h, gamma, eps, router, E, k, renorm, has_gate=has_gate, align=2 if rep == 2 else None)
        assert got is not None
        x, ids, w, gate, sort = got
        assert (sort is None) == (rep < 2)
        if sort is not None:
            for i, (mine, theirs) in enumerate(zip(sort, ops.moe_align(ids, E, always=2))):
                n_set = T * k if i == 3 else mine.numel()           # the inverse map covers the pairs only
                assert torch.equal(mine[:n_set], theirs[:n_set]), "the launch's own sort is that of moe_align"
        # the same formula as the norm kernel: at most the last float32 bit differs, which moves a
        # bfloat16 result only where it stands on a rounding boundary
        differ = x != x_sep
        assert int(differ.sum()) <= max(1, x.numel() // 10000), "the fused norm rounds like the norm kernel"
        assert bool(((x.float() - x_sep.float()).abs() <= x_sep.float().abs() * 2.0 ** -7).all())
        want_x = plain.rms_norm(h.double().cpu(), gamma.double().cpu(), eps)
        close(x, want_x, torch.bfloat16, "normed rows")
        logits = router.double().cpu() @ x.double().cpu().T                  # [E(+1), T]
        for t in range(T):
            want_ids, want_w = plain.route_top_k(logits[:E, t], k, renorm)
            assert ids[t].tolist() == want_ids, f"rep {rep} token {t}: experts {ids[t].tolist()} != {want_ids}"
            close(w[t], want_w, torch.float32, f"router weights token {t}")
        if has_gate:
            close(gate, torch.sigmoid(logits[E]), torch.float32, "shared gate")
    assert int(ops._counter(DEV).abs().sum()) == 0
    assert ops.moe_front(rnd(257, H), gamma, eps, router, E, k, renorm, has_gate=has_gate) is None     # too many rows


@pytest.mark.parametrize("T,E,k", [(5000, 60, 4), (3000, 700, 2), (1, 3, 1), (130, 1, 1), (2048, 60, 4), (701, 7, 3), (683, 5, 3)])
def test_sort_by_expert_at_large_sizes(T, E, k):
    """more pairs than one round of counters holds: rows of several groups; against a stable sort"""
    from ferrox_amd import ops
    g = torch.Generator().manual_seed(T + E)
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32).to(DEV)
    offsets, sorted_token, sorted_pair, inv = ops.moe_align(ids, E)
    flat = ids.flatten().long().cpu()
    order = torch.sort(flat, stable=True).indices
    assert sorted_pair.cpu().tolist() == order.tolist()
    assert sorted_token.cpu().tolist() == (order // k).tolist()
    assert offsets.cpu().tolist() == [0] + torch.cumsum(torch.bincount(flat, minlength=E), 0).tolist()
    assert inv.cpu()[order].tolist() == list(range(T * k))


@pytest.mark.parametrize("T,E,k,S", [(24, 60, 4, 4), (64, 8, 2, 3), (17, 5, 1, 1), (40, 6, 3, 2)])
def test_sort_by_expert_with_experts_that_every_token_takes(T, E, k, S):
    """S further experts behind the sorted pairs, each with all T tokens as its rows (a shared expert cut into
    pieces), and the grouped products over that layout against one product per expert"""
    from ferrox_amd import ops
    g = torch.Generator().manual_seed(T + E)
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32).to(DEV)
    plain_sort = ops.moe_align(ids, E)
    offsets, sorted_token, sorted_pair, _ = ops.moe_align(ids, E, always=S)
    n = T * k
    assert offsets.cpu().tolist() == plain_sort[0].cpu().tolist() + [n + (s + 1) * T for s in range(S)]
    assert sorted_token.cpu().tolist() == plain_sort[1].cpu().tolist() + list(range(T)) * S
    assert sorted_pair.cpu().tolist() == plain_sort[2].cpu().tolist() + list(range(n, n + S * T))
    H, I = 64, 32
    x = rnd(T, H, dtype=torch.bfloat16)
    w_gu, w_dn = rnd(E + S, 2 * I, H, dtype=torch.bfloat16, seed=1, scale=0.3), rnd(E + S, H, I, dtype=torch.bfloat16, seed=2, scale=0.3)
    act = ops.gemm(x, w_gu, epilogue=ops.EPI_GATED, a_rows=sorted_token, expert_offsets=offsets, n_rows=n + S * T)
    y = ops.gemm(act, w_dn, epilogue=ops.EPI_STORE_F32, expert_offsets=offsets, c_rows=sorted_pair)
    assert y.shape == (n + S * T, H)
    xd = x.double().cpu()
    for s_ in range(S):                      # piece s: every token through expert E + s
        e = E + s_
        a = (plain.silu(xd @ w_gu[e, :I].double().cpu().T) * (xd @ w_gu[e, I:].double().cpu().T)).to(torch.bfloat16).double()
        close(y[n + s_ * T:n + (s_ + 1) * T], a @ w_dn[e].double().cpu().T, torch.bfloat16, f"piece {s_}")
    t, j = 3 % T, k - 1                      # and a routed pair
    e = int(ids[t, j])
    a = (plain.silu(xd[t] @ w_gu[e, :I].double().cpu().T) * (xd[t] @ w_gu[e, I:].double().cpu().T)).to(torch.bfloat16).double()
    close(y[t * k + j], a @ w_dn[e].double().cpu().T, torch.bfloat16, "a routed pair")


@pytest.mark.parametrize("T,E,k", [(1, 8, 2), (8, 60, 4), (64, 60, 4), (33, 130, 8), (65, 6, 3), (300, 60, 4)])
def test_route_in_one_launch_equals_two(T, E, k):
    """selection and sort fused for small batches give what the two kernels give"""
    from ferrox_amd import ops
    logits = rnd(T, E + 1, scale=2.0)
    fused = ops.route(logits, E, k, True, has_gate=True)
    ids, w, gate = ops.router_select(logits, E, k, True, has_gate=True)
    two = (ids, w, gate) + ops.moe_align(ids, E)
    for a, b in zip(fused, two):
        assert torch.equal(a, b)


def test_tokens_fed_from_sampled_ids():
    """tokens[place] = ids[row] for the pairs given, everything else untouched; buffers of the wrong kind are refused"""
    from ferrox_amd import ops
    g = torch.Generator().manual_seed(3)
    tokens = torch.randint(0, 1000, (777,), generator=g, dtype=torch.int32)
    ids = torch.randint(0, 1000, (300,), generator=g, dtype=torch.int32)
    places = torch.randperm(777, generator=g)[:300]
    rows = torch.randint(0, 300, (300,), generator=g)
    expect = tokens.clone()
    expect[places] = ids[rows]
    d_tokens, pairs = tokens.cuda(), torch.stack([places, rows], 1).to(torch.int32).cuda()
    ops.feed_tokens(d_tokens, ids.cuda(), pairs, 777, 300)
    assert torch.equal(d_tokens.cpu(), expect)
    with pytest.raises(ops.KernelError):
        ops.feed_tokens(d_tokens, ids.cuda().long(), pairs, 777, 300)
    with pytest.raises(ops.KernelError):
        ops.feed_tokens(d_tokens, ids.cuda(), pairs, 778, 300)


@pytest.mark.parametrize("T,E,k,I,H", [(40, 4, 2, 64, 128), (100, 4, 2, 128, 192), (24, 6, 3, 64, 64)])
def test_sorted_experts_through_either_product(T, E, k, I, H):
    """rows sorted by expert, more than three an expert: the tiled product takes them by itself; the product for few
    rows, told to (it takes up to 64 rows an expert), gives the same activations and outputs up to rounding, and
    both agree with per-token loops"""
    from ferrox_amd import debug, ops
    dtype = torch.bfloat16
    x = rnd(T, H, dtype=dtype)
    w_gu, w_dn = rnd(E, 2 * I, H, dtype=dtype, seed=1, scale=0.3), rnd(E, H, I, dtype=dtype, seed=2, scale=0.3)
    g = torch.Generator().manual_seed(7)
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32).to(DEV)
    offsets, sorted_token, sorted_pair, inv = ops.moe_align(ids, E)
    xd, gud, dnd = x.double().cpu(), w_gu.double().cpu(), w_dn.double().cpu()
    ref = torch.zeros(T * k, H, dtype=torch.float64)
    for t in range(T):
        for j in range(k):
            e = int(ids[t, j])
            a = (plain.silu(xd[t] @ gud[e, :I].T) * (xd[t] @ gud[e, I:].T)).to(torch.bfloat16).double()
            ref[t * k + j] = a @ dnd[e].T
    outs = []
    for few in (3, 64):
        with debug.kernel_switch("gemm", "few_rows", few):
            act = ops.gemm(x, w_gu, epilogue=ops.EPI_GATED, a_rows=sorted_token, expert_offsets=offsets, n_rows=T * k)
            y = ops.gemm(act, w_dn, epilogue=ops.EPI_STORE_F32, expert_offsets=offsets, c_rows=sorted_pair)
        close(y, ref, dtype, f"sorted experts, few_rows {few}", k=I)
        outs.append(y)
    assert float((outs[0] - outs[1]).abs().max()) <= 2e-2 * float(ref.abs().max())
