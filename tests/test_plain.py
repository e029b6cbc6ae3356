"""What fixes the plain implementation beside the reference's text: vectors that the reference's own
tests hold, special cases that reduce to a library routine, and invariants.  Each is chosen so that
a plausible mistake (a wrong sign or pairing, a norm in the wrong place) fails it."""
import math

import pytest
import torch

import plain_qwen2moe as plain
from conftest import TINY_A, TINY_B

torch.manual_seed(0)
D = torch.float64


def randn(*shape):
    return torch.randn(*shape, dtype=D)


# ---- RMSNorm -----------------------------------------------------------------
def test_rms_norm_against_library_formula_and_reference_vector():
    x, w = randn(5, 24), randn(24)
    want = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-5) * w
    assert torch.allclose(plain.rms_norm(x, w, 1e-5), want, atol=1e-12)
    # ferrox-core/src/matmul.rs:376-383: [3, 4] with unit weight keeps its direction, rms becomes 1
    y = plain.rms_norm(torch.tensor([3.0, 4.0], dtype=D), torch.ones(2, dtype=D), 0.0)
    assert torch.allclose(y, torch.tensor([3.0, 4.0], dtype=D) / math.sqrt(12.5))
    assert torch.allclose(plain.rms_norm(7.0 * x, w, 1e-12), plain.rms_norm(x, w, 1e-12), atol=1e-9)   # scale-free
    # eps inside the root: a zero vector stays zero and finite; "1 + w" would not map w=0 to 0
    assert torch.equal(plain.rms_norm(torch.zeros(4, dtype=D), torch.ones(4, dtype=D), 1e-6), torch.zeros(4, dtype=D))
    assert torch.equal(plain.rms_norm(x, torch.zeros(24, dtype=D), 1e-6), torch.zeros(5, 24, dtype=D))


# ---- rotary ----------------------------------------------------------------
def test_rope_pairing_sign_and_frequencies():
    # dim 4, theta 100, position 1: pair (0, 2) turns by 1 rad, pair (1, 3) by 1/10 rad
    v = torch.tensor([1.0, 0.0, 0.0, 1.0], dtype=D)
    got = plain.rope_neox(v, 1, 100.0)
    want = torch.tensor([math.cos(1.0), -math.sin(0.1), math.sin(1.0), math.cos(0.1)], dtype=D)
    assert torch.allclose(got, want, atol=1e-12)
    x = randn(3, 16)
    assert torch.equal(plain.rope_neox(x, 0, 1e4), x)                                   # attention.rs:815-830
    assert torch.allclose(plain.rope_neox(x, 9, 1e4).norm(dim=-1), x.norm(dim=-1))       # a rotation
    assert torch.allclose(plain.rope_neox(plain.rope_neox(x, 9, 1e4), -9, 1e4), x, atol=1e-12)
    # adjacent-pair layout is a different function when dim > 2 (attention.rs:900-936)
    inter = x.clone()
    for i in range(8):
        a, b, ang = x[:, 2 * i], x[:, 2 * i + 1], 9 / (1e4 ** (2 * i / 16))
        inter[:, 2 * i], inter[:, 2 * i + 1] = a * math.cos(ang) - b * math.sin(ang), a * math.sin(ang) + b * math.cos(ang)
    assert not torch.allclose(plain.rope_neox(x, 9, 1e4), inter, atol=1e-3)


def test_rope_angle_in_float32_is_one_rounded_product():
    """attention.rs:26-27: `angle = pos as f32 * freq` with a float32 frequency.  The float32 angle is the rounded
    product of the rounded frequency, equal to the exact angle where nothing is rounded (pair 0, whose frequency
    is 1) and within half a unit in the last place of the angle, plus the frequency's own rounding, elsewhere."""
    import numpy as np
    for theta, dim in ((1e4, 16), (1e6, 128)):
        for pos in (0, 1, 7, 500, 2047, 2048, 32767):
            assert plain.rope_angle(pos, 0, dim, theta, "float32") == float(pos)
            for i in (1, 3, dim // 2 - 1):
                exact, f32 = plain.rope_angle(pos, i, dim, theta), plain.rope_angle(pos, i, dim, theta, "float32")
                assert f32 == float(np.float32(f32))                            # a float32 number
                assert abs(f32 - exact) <= 2.0 ** -23 * abs(exact) + 1e-300
    # deep in a sequence the two are apart by far more than the tests' float32 tolerance
    assert max(abs(plain.rope_angle(2047, i, 16, 1e4, "float32") - plain.rope_angle(2047, i, 16, 1e4)) for i in range(8)) > 1e-6
    x = randn(16)
    near = plain.rope_neox(x, 2047, 1e4, "float32")
    assert torch.allclose(near, plain.rope_neox(x, 2047, 1e4), atol=1e-3) and not torch.allclose(
        near, plain.rope_neox(x, 2047, 1e4), atol=1e-7)


def test_rope_scores_depend_on_distance_only():
    q, k = randn(16), randn(16)
    a = plain.rope_neox(q, 37, 1e6) @ plain.rope_neox(k, 30, 1e6)
    b = plain.rope_neox(q, 107, 1e6) @ plain.rope_neox(k, 100, 1e6)
    c = plain.rope_neox(q, 37, 1e6) @ plain.rope_neox(k, 31, 1e6)
    assert abs(float(a - b)) < 1e-9 and abs(float(a - c)) > 1e-6


# ---- attention ------------------------------------------------------------------
def test_attention_against_library_sdpa():
    T, nh, nkv, hd = 9, 4, 2, 8
    q, k, v = randn(T, nh, hd), randn(T, nkv, hd), randn(T, nkv, hd)
    got = plain.causal_attention(q, k, v, nh, nkv, None)
    kk, vv = k.repeat_interleave(nh // nkv, 1), v.repeat_interleave(nh // nkv, 1)      # consecutive q heads share
    want = torch.nn.functional.scaled_dot_product_attention(q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1),
                                                            is_causal=True).transpose(0, 1)
    assert torch.allclose(got, want, atol=1e-12)


def test_attention_special_cases():
    nh, nkv, hd = 4, 2, 8
    q, k, v = randn(6, nh, hd), randn(6, nkv, hd), randn(6, nkv, hd)
    out = plain.causal_attention(q, k, v, nh, nkv, None)
    # a single position returns v (attention.rs:974-983); heads 0,1 -> kv 0 and 2,3 -> kv 1 (986-1004)
    for h in range(nh):
        assert torch.allclose(out[0, h], v[0, h // 2])
    assert torch.equal(plain.causal_attention(q, k, v, nh, nkv, 6), out)                  # window >= length
    assert torch.equal(plain.causal_attention(q, k, v, nh, nkv, 100), out)
    w1 = plain.causal_attention(q, k, v, nh, nkv, 1)                                       # window 1: own v (1076-1089)
    for t in range(6):
        for h in range(nh):
            assert torch.allclose(w1[t, h], v[t, h // 2])
    # window 3 at position 5 sees exactly positions 3, 4, 5
    w3 = plain.causal_attention(q, k, v, nh, nkv, 3)
    ref = plain.causal_attention(q[3:], k[3:], v[3:], nh, nkv, None)
    assert torch.allclose(w3[5], ref[2])
    # one score made to stand out picks that key's value
    q2, k2 = torch.zeros(6, nh, hd, dtype=D), torch.zeros(6, nkv, hd, dtype=D)
    q2[5, :, 0], k2[2, :, 0] = 100.0, 100.0
    far = plain.causal_attention(q2, k2, v, nh, nkv, None)
    assert torch.allclose(far[5, 3], v[2, 1], atol=1e-9)
    assert not torch.allclose(plain.causal_attention(q2, k2, v, nh, nkv, 3)[5, 3], v[2, 1], atol=1e-3)   # outside the window


# ---- router and experts ---------------------------------------------------------
def test_router_vectors_of_the_reference():
    ids, w = plain.route_top_k(torch.tensor([0.1, 5.0, 0.2, 3.0, -1.0], dtype=D), 2, True)     # lib.rs:834-841
    assert ids == [1, 3] and abs(float(w.sum()) - 1.0) < 1e-12
    ids, w = plain.route_top_k(torch.arange(1, 9, dtype=D), 3, False)                           # lib.rs:863-893
    assert ids == [7, 6, 5]
    assert torch.allclose(w, torch.tensor([0.6323223, 0.2326232, 0.0855683], dtype=D), atol=1e-4)
    assert abs(float(w.sum()) - 0.9505138) < 1e-4
    ids2, w2 = plain.route_top_k(torch.arange(1, 9, dtype=D), 3, True)
    assert ids2 == ids and torch.allclose(w2, w / w.sum())
    logits = randn(6)
    ids, w = plain.route_top_k(logits, 6, False)                  # k = E without renormalisation: the softmax itself
    assert torch.allclose(w, torch.softmax(logits, 0)[ids]) and abs(float(w.sum()) - 1) < 1e-12
    assert plain.route_top_k(torch.zeros(5, dtype=D), 2, False)[0] == [0, 1]                   # ties: lower index


def test_combine_vector_of_the_reference():
    out = plain.combine_expert_outputs([(torch.tensor([2.0, 2.0], dtype=D), 0.5), (torch.tensor([4.0, 4.0], dtype=D), 0.5)],
                                       [torch.tensor([1.0, 1.0], dtype=D)], 2)                  # lib.rs:1162-1168
    assert torch.equal(out, torch.tensor([4.0, 4.0], dtype=D))


def test_swiglu_and_moe_special_cases():
    H, I, E = 12, 20, 4
    x = randn(H)
    g, u, d = randn(I, H), randn(I, H), randn(H, I)
    dense = plain.swiglu_mlp(x, g, u, d)
    assert torch.allclose(dense, (torch.nn.functional.silu(g @ x) * (u @ x)) @ d.T, atol=1e-12)
    assert float(plain.silu(torch.tensor(0.0, dtype=D))) == 0.0                                 # matmul.rs:343-350
    router = randn(E, H)
    same = [(g, u, d)] * E
    # identical experts with renormalised weights are one dense MLP; without renormalisation scaled by the mass
    assert torch.allclose(plain.moe_ffn_token(x, router, same, 2, True, None, None), dense, atol=1e-12)
    _, w = plain.route_top_k(router @ x, 2, False)
    assert torch.allclose(plain.moe_ffn_token(x, router, same, 2, False, None, None), dense * w.sum(), atol=1e-12)
    # one expert, top-1: the dense layer (decoder.rs:2390-2402)
    assert torch.allclose(plain.moe_ffn_token(x, randn(1, H), [(g, u, d)], 1, False, None, None), dense, atol=1e-12)
    # k = E without renormalisation: the softmax mixture of all experts
    experts = [(randn(I, H), randn(I, H), randn(H, I)) for _ in range(E)]
    p = torch.softmax(router @ x, 0)
    mix = sum(p[e] * plain.swiglu_mlp(x, *experts[e]) for e in range(E))
    assert torch.allclose(plain.moe_ffn_token(x, router, experts, E, False, None, None), mix, atol=1e-12)
    # shared expert: gate weights 0 give the factor 1/2; in general sigmoid(w . x) (decoder.rs:3994-4057)
    sh = (randn(I, H), randn(I, H), randn(H, I))
    routed = plain.moe_ffn_token(x, router, experts, 2, True, None, None)
    assert torch.allclose(plain.moe_ffn_token(x, router, experts, 2, True, sh, torch.zeros(1, H, dtype=D)),
                          routed + 0.5 * plain.swiglu_mlp(x, *sh), atol=1e-12)
    gw = randn(1, H)
    assert torch.allclose(plain.moe_ffn_token(x, router, experts, 2, True, sh, gw),
                          routed + torch.sigmoid((gw[0] * x).sum()) * plain.swiglu_mlp(x, *sh), atol=1e-12)


# ---- whole model ----------------------------------------------------------------
@pytest.fixture(scope="module")
def tiny(model_folders):
    return {n: plain.load_folder(model_folders(n, "float32")) for n in ("A", "B")}


def test_layer_plan_and_windows():
    assert [plain.layer_is_sparse(TINY_A, l) for l in range(2)] == [True, True]
    assert [plain.layer_is_sparse(TINY_B, l) for l in range(3)] == [False, True, False]
    assert [plain.layer_window(TINY_B, l) for l in range(3)] == [None, 16, 16]
    assert [plain.layer_window(TINY_A, l) for l in range(2)] == [None, None]


def test_positions_shift_invariance(tiny):
    """Only distances count (rotary, causal mask, window): shifting every position changes nothing."""
    for name in ("A", "B"):
        cfg, w = tiny[name]
        toks = [5, 17, 3, 99, 42, 7, 7, 1, 250, 33, 12, 8, 90, 21, 60, 2, 4, 6, 19, 55]
        a = plain.forward(cfg, w, toks, angles="exact")
        b = plain.forward(cfg, w, toks, start_pos=37, angles="exact")
        assert torch.allclose(a, b, atol=1e-9), name
        # with the reference's float32 angles the shifted run differs by their rounding alone
        c = plain.forward(cfg, w, toks, start_pos=37)
        assert torch.allclose(a, c, atol=1e-6) and not torch.equal(b, c), name


def test_prefix_property_and_bias_is_live(tiny):
    cfg, w = tiny["B"]
    toks = list(range(40, 70))
    full = plain.forward(cfg, w, toks)
    assert torch.allclose(plain.forward(cfg, w, toks[:11]), full[:11], atol=1e-10)             # causal
    # the window matters beyond its length (layers 1, 2 have W = 16) ...
    no_window = dict(cfg, use_sliding_window=False)
    wide = plain.forward(no_window, w, toks)
    assert torch.allclose(wide[:16], full[:16], atol=1e-10) and not torch.allclose(wide[20:], full[20:], atol=1e-6)
    # ... the bias changes the output from position 1 on (position 0 attends to itself only: decoder.rs:4414-4450)
    w0 = dict(w)
    for l in range(cfg["num_hidden_layers"]):
        for n in ("q", "k"):
            w0[f"model.layers.{l}.self_attn.{n}_proj.bias"] = torch.zeros_like(w[f"model.layers.{l}.self_attn.{n}_proj.bias"])
    nob = plain.forward(cfg, w0, toks)
    assert torch.allclose(nob[0], full[0], atol=1e-10) and not torch.allclose(nob[1:], full[1:], atol=1e-7)
    # tied head == explicit copy of the embedding
    untied = dict(cfg, tie_word_embeddings=False)
    w1 = dict(w, **{"lm_head.weight": w["model.embed_tokens.weight"]})
    assert torch.equal(plain.forward(untied, w1, toks), full)


# ---- the block's wiring --------------------------------------------------------
WIRING = {"num_hidden_layers": 2, "hidden_size": 24, "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 8,
          "num_experts": 3, "num_experts_per_tok": 2, "norm_topk_prob": False, "moe_intermediate_size": 10,
          "shared_expert_intermediate_size": 12, "intermediate_size": 14, "decoder_sparse_step": 1,
          "mlp_only_layers": [1], "vocab_size": 40, "rope_theta": 100.0, "rms_norm_eps": 1e-30,
          "use_sliding_window": False, "tie_word_embeddings": False}


def wiring_weights(cfg, scale=0.4):
    """random tensors under the checkpoint's names (layer 0 sparse with a shared expert, layer 1 dense)"""
    g = torch.Generator().manual_seed(11)
    r = lambda *shape: torch.randn(*shape, dtype=D, generator=g) * scale
    H, hd = cfg["hidden_size"], cfg["head_dim"]
    qw, kvw = cfg["num_attention_heads"] * hd, cfg["num_key_value_heads"] * hd
    w = {"model.embed_tokens.weight": r(cfg["vocab_size"], H), "lm_head.weight": r(cfg["vocab_size"], H),
         "model.norm.weight": 1 + r(H)}
    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}."
        w[p + "input_layernorm.weight"], w[p + "post_attention_layernorm.weight"] = 1 + r(H), 1 + r(H)
        for n, rows in (("q", qw), ("k", kvw), ("v", kvw)):
            w[p + f"self_attn.{n}_proj.weight"], w[p + f"self_attn.{n}_proj.bias"] = r(rows, H), r(rows)
        w[p + "self_attn.o_proj.weight"] = r(H, qw)
        if plain.layer_is_sparse(cfg, l):
            I, S = cfg["moe_intermediate_size"], cfg["shared_expert_intermediate_size"]
            w[p + "mlp.gate.weight"] = r(cfg["num_experts"], H)
            for e in range(cfg["num_experts"]):
                for n, shape in (("gate", (I, H)), ("up", (I, H)), ("down", (H, I))):
                    w[p + f"mlp.experts.{e}.{n}_proj.weight"] = r(*shape)
            for n, shape in (("gate", (S, H)), ("up", (S, H)), ("down", (H, S))):
                w[p + f"mlp.shared_expert.{n}_proj.weight"] = r(*shape)
            w[p + "mlp.shared_expert_gate.weight"] = r(1, H)
        else:
            I = cfg["intermediate_size"]
            for n, shape in (("gate", (I, H)), ("up", (I, H)), ("down", (H, I))):
                w[p + f"mlp.{n}_proj.weight"] = r(*shape)
    return w


WIRING_TOKENS = [3, 17, 5, 5, 39, 0, 21, 8, 30, 11, 2]


def test_norms_stand_before_the_sublayers():
    """Pre-norm (ferrox-models/src/decoder.rs:1-5, 2155-2173): every sublayer reads norm(h) and adds into h, so
    scaling what enters the residual stream (the embedding and each sublayer's last matrix) by c scales h by c
    everywhere and leaves the logits alone (eps -> 0).  A norm after a sublayer, a sublayer that reads h itself,
    or a residual taken from the normed rows would each break this."""
    w = wiring_weights(WIRING)
    base = plain.forward(WIRING, w, WIRING_TOKENS)
    into_stream = [n for n in w if n == "model.embed_tokens.weight" or n.endswith("o_proj.weight")
                   or n.endswith("down_proj.weight")]
    assert len(into_stream) == 1 + 2 + 3 + 1 + 1
    scaled = {n: (t * 7.5 if n in into_stream else t) for n, t in w.items()}
    assert torch.allclose(plain.forward(WIRING, scaled, WIRING_TOKENS), base, atol=1e-9)
    # and each of them matters: scaling one alone changes the logits
    for n in into_stream:
        one = dict(w, **{n: w[n] * 7.5})
        assert not torch.allclose(plain.forward(WIRING, one, WIRING_TOKENS), base, atol=1e-6), n
    # the final norm is applied (scaling the last layer's output alone would otherwise scale the logits)
    assert float(base.abs().max()) < 1e3


def test_values_are_not_rotated_and_queries_are_rotated_whole():
    """With zero q and k every score is zero, attention is the running mean of the values, and those are
    W_v x + b_v as they are: no rotation (ferrox-models/src/decoder.rs:2106-2111 rotates q and k only), head h
    of the output reading kv head h // group (ferrox-core/src/attention.rs:432-438).  And with q and k back, the
    rotation covers the whole head: changing the last pair's partner dimension changes the scores."""
    cfg = dict(WIRING, num_hidden_layers=1, mlp_only_layers=[0])
    w = wiring_weights(cfg)
    p = "model.layers.0."
    for n in ("q", "k"):
        w[p + f"self_attn.{n}_proj.weight"] = torch.zeros_like(w[p + f"self_attn.{n}_proj.weight"])
        w[p + f"self_attn.{n}_proj.bias"] = torch.zeros_like(w[p + f"self_attn.{n}_proj.bias"])
    T, H, nh, nkv, hd = len(WIRING_TOKENS), 24, 4, 2, 8
    h = w["model.embed_tokens.weight"][torch.tensor(WIRING_TOKENS)]
    x = plain.rms_norm(h, w[p + "input_layernorm.weight"], 1e-30)
    v = (x @ w[p + "self_attn.v_proj.weight"].T + w[p + "self_attn.v_proj.bias"]).reshape(T, nkv, hd)
    mean = torch.cumsum(v, 0) / torch.arange(1, T + 1, dtype=D)[:, None, None]
    a = torch.stack([mean[:, hh // (nh // nkv)] for hh in range(nh)], dim=1)            # [T, nh, hd], head-major
    h = h + a.reshape(T, nh * hd) @ w[p + "self_attn.o_proj.weight"].T
    x2 = plain.rms_norm(h, w[p + "post_attention_layernorm.weight"], 1e-30)
    h = h + plain.swiglu_mlp(x2, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    want = plain.rms_norm(h, w["model.norm.weight"], 1e-30) @ w["lm_head.weight"].T
    assert torch.allclose(plain.forward(cfg, w, WIRING_TOKENS), want, atol=1e-10)
    # rotation over the whole head: q = k = one-hot in the last dimension of the first half of head 0 and
    # its partner (dimension hd-1); a rotation of fewer dimensions would leave these scores position-free
    w = wiring_weights(cfg)
    q, k = torch.zeros(T, nh, hd, dtype=D), torch.zeros(T, nkv, hd, dtype=D)
    q[:, :, hd // 2 - 1] = 1.0
    k[:, :, hd // 2 - 1] = 1.0
    rq, rk = plain.rope_neox_rows(q, range(T), 100.0), plain.rope_neox_rows(k, range(T), 100.0)
    assert float(rq[5, 0, hd - 1].abs()) > 1e-3                                         # the pair (hd/2-1, hd-1) turns
    s = torch.einsum("td,sd->ts", rq[:, 0], rk[:, 0])
    assert abs(float(s[9, 2] - s[8, 1])) < 1e-12 and abs(float(s[9, 2] - s[9, 3])) > 1e-6


def test_heads_are_concatenated_head_major():
    """Permuting whole heads of q, k and v together with the matching column blocks of o_proj changes nothing
    (ferrox-models/src/decoder.rs:2150-2157: the heads' outputs lie one after the other); a concat that
    interleaves the heads' dimensions would not survive it.  Permuting the column blocks alone does change it."""
    cfg, w = WIRING, wiring_weights(WIRING)
    base = plain.forward(cfg, w, WIRING_TOKENS)
    nh, nkv, hd = 4, 2, 8
    group = nh // nkv
    kv_perm = [1, 0]
    q_perm = [kv_perm[hh // group] * group + hh % group for hh in range(nh)]             # q heads follow their kv head
    rows = lambda perm: torch.cat([torch.arange(hh * hd, (hh + 1) * hd) for hh in perm])
    moved, only_o = dict(w), dict(w)
    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}.self_attn."
        for n, perm in (("q", q_perm), ("k", kv_perm), ("v", kv_perm)):
            moved[p + f"{n}_proj.weight"] = w[p + f"{n}_proj.weight"][rows(perm)]
            moved[p + f"{n}_proj.bias"] = w[p + f"{n}_proj.bias"][rows(perm)]
        moved[p + "o_proj.weight"] = w[p + "o_proj.weight"][:, rows(q_perm)]
        only_o[p + "o_proj.weight"] = w[p + "o_proj.weight"][:, rows(q_perm)]
    assert torch.allclose(plain.forward(cfg, moved, WIRING_TOKENS), base, atol=1e-10)
    assert not torch.allclose(plain.forward(cfg, only_o, WIRING_TOKENS), base, atol=1e-6)


# ---- sampler ----------------------------------------------------------------
def test_xorshift_stream():
    r = plain.XorShift64(1)
    assert r.next_u64() == 0x40822041                 # 1 -> 0x2001 -> 0x2041 -> 0x40822041 with shifts 13, 7, 17
    assert plain.XorShift64(0).state == 0x9E3779B97F4A7C15          # sampling.rs:66-72
    r = plain.XorShift64(12345)
    xs = [r.next_f32() for _ in range(1000)]
    assert all(0.0 <= x < 1.0 for x in xs) and 0.4 < sum(xs) / 1000 < 0.6


def test_sampler_special_cases():
    logits = torch.randn(50).tolist()
    best = max(range(50), key=lambda i: logits[i])
    for seed in range(5):
        assert plain.sample(logits, plain.XorShift64(seed)) == best                                  # greedy
        assert plain.sample(logits, plain.XorShift64(seed), temperature=0.9, top_k=1) == best         # sampling.rs:241-381
        assert plain.sample(logits, plain.XorShift64(seed), temperature=0.9, top_p=1e-9) == best
    a = [plain.sample(logits, plain.XorShift64(7), temperature=1.0) for _ in range(3)]
    assert a[0] == a[1] == a[2]                                                                       # same seed, same draw
    counts = {}
    rng = plain.XorShift64(3)
    for _ in range(300):
        t = plain.sample(logits, rng, temperature=1.0, top_k=3)
        counts[t] = counts.get(t, 0) + 1
    assert set(counts) <= set(sorted(range(50), key=lambda i: -logits[i])[:3])
    # repetition penalty pushes a repeated favourite down (greedy)
    assert plain.sample(logits, plain.XorShift64(0), repetition_penalty=1e6, history=[best]) != best
    assert plain.argmax_first([1.0, 3.0, 3.0]) == 1
