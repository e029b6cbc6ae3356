"""Parts alone and put together from data: each built-in part in a model of its own beside
stand-in parts defined here, a mixer with state of its own registered from outside the package,
layer orders that name a layer twice or read another layer's cache."""
import math
import os

import pytest
import torch

import plain_qwen2moe as plain
import replay_util as ru
from ferrox_amd import ops
from ferrox_amd.engine.model import Model
from ferrox_amd.engine.runner import ModelRunner, StepEntry
from ferrox_amd.parts import (FEED_FORWARDS, MIXERS, POSITION_ENCODINGS, FeedForward, LayerSpec, Mixer, ModelSpec,
                              ParamSpec, PartSpec, PositionEncoding, Rotary, ScheduleEntry)
from ferrox_amd.weights import RandomSource

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


# ---- stand-ins, defined outside the package -----------------------------------------
@FEED_FORWARDS.register("test_no_ffn")
class NoFFN(FeedForward):
    def __init__(self, hidden_size: int = 0):
        pass

    def forward(self, x, ctx, residual):
        return None


@MIXERS.register("test_no_mixer")
class NoMixer(Mixer):
    def __init__(self, hidden_size: int = 0):
        pass

    def forward(self, x, ctx, cache, residual):
        return None


@MIXERS.register("test_running_mean")
class RunningMean(Mixer):
    """y_t = W * mean(x_0 .. x_t): a mixer whose whole memory is a fixed-size state per request
    (the running sum), kept in a state slot; written with torch operations."""

    def __init__(self, hidden_size: int):
        self.hidden_size = hidden_size
        self.weight = None

    def param_specs(self):
        return {"mix.weight": ParamSpec((self.hidden_size, self.hidden_size))}

    def load(self, fetch):
        self.weight = fetch("mix.weight")

    def state_shapes(self):
        return {"sum": ((self.hidden_size,), torch.float32)}

    def forward(self, x, ctx, cache, residual):
        state = cache.state["sum"]
        for s in range(ctx.n_seqs):
            b, e = ctx.q_starts[s], ctx.q_starts[s + 1]
            run = state[ctx.slots[s]] + torch.cumsum(x[b:e].float(), 0)
            state[ctx.slots[s]] = run[-1]
            mean = run / (ctx.positions[b:e].float()[:, None] + 1.0)
            y = mean.to(self.weight.dtype) @ self.weight.T
            ops.residual_add(residual[b:e], y.contiguous())


@MIXERS.register("test_window_mean")
class WindowMean(Mixer):
    """y_t = W * mean(x_s for t - span < s <= t): a mixer that keeps its inputs in pages of a cache group of its
    own, which ages by a window; written with torch operations on device tensors only, so that a decode step can
    be recorded (`graph_safe`): nothing is read from the context's host lists, every index comes from
    `positions`, `token_seq` and the block table."""
    graph_safe = True

    def __init__(self, hidden_size: int, span: int):
        self.hidden_size, self.span, self.window = hidden_size, span, span
        self.weight = None

    def param_specs(self):
        return {"mix.weight": ParamSpec((self.hidden_size, self.hidden_size))}

    def load(self, fetch):
        self.weight = fetch("mix.weight")

    def cache_group(self):
        return ("test_window_mean", self.span), self.span

    def page_shapes(self, block_size):
        return {"x": (block_size, self.hidden_size)}

    def forward(self, x, ctx, cache, residual):
        pages, table, bs = cache.pages["x"], ctx.block_tables[cache.group], cache.block_size
        pos, seq = ctx.positions.long(), ctx.token_seq.long()
        pages[table[seq, pos // bs].long(), pos % bs] = x                                  # write, then read
        back = pos[:, None] - torch.arange(self.span, device=x.device)[None, :]           # [T, span] positions read
        seen = back >= 0
        back = back.clamp_min(0)
        rows = pages[table[seq[:, None], back // bs].long(), back % bs].float()            # [T, span, H]
        mean = (rows * seen[:, :, None]).sum(1) / seen.sum(1, keepdim=True)
        ops.residual_add(residual, (mean.to(self.weight.dtype) @ self.weight.T).contiguous())


@POSITION_ENCODINGS.register("test_banded_rope")
class BandedRope(PositionEncoding):
    """Split-half rotary whose pair i turns slower by a factor of its own, 1 + 8 |b_i| with b a tensor of the
    checkpoint: the kernels rotate, the part only hands them the table."""

    def __init__(self, head_dim: int, theta: float):
        self.head_dim, self.theta = head_dim, theta
        self.factors = None

    def param_specs(self):
        return {"bands": ParamSpec((self.head_dim // 2,))}

    def load(self, fetch):
        self.factors = (1.0 + 8.0 * fetch("bands").float().abs()).contiguous()

    def rotary(self):
        return Rotary(self.head_dim, self.theta, False, self.factors)


@POSITION_ENCODINGS.register("test_decay_positions")
class DecayPositions(PositionEncoding):
    """Not a rotation: q_t is scaled by g^t and k_s by g^-s per head dimension, with a gain g of its own
    (a tensor of the checkpoint), so that a score carries g^(t-s).  Each token is scaled by its own
    position only, which is what lets keys be cached.  Written with torch operations."""

    def __init__(self, head_dim: int):
        self.head_dim = head_dim
        self.gain = None

    def param_specs(self):
        return {"gain": ParamSpec((self.head_dim,))}

    def load(self, fetch):
        self.gain = fetch("gain")

    @staticmethod
    def factors(gain, positions):
        """[T, head_dim] of g^t with g = 1 + gain / 64 (float32)"""
        return torch.exp(positions.float()[:, None] * torch.log1p(gain.float() / 64.0)[None, :])

    def apply(self, q, k, ctx):
        f = self.factors(self.gain, ctx.positions)
        hd = self.head_dim
        qv, kv = q.view(q.shape[0], -1, hd), k.view(k.shape[0], -1, hd)
        qv.copy_((qv.float() * f[:, None, :]).to(q.dtype))
        kv.copy_((kv.float() / f[:, None, :]).to(k.dtype))


@FEED_FORWARDS.register("test_top1_ffn")
class Top1Linear(FeedForward):
    """y = sigmoid(r_e) * W_e x for the one expert e with the largest router logit r = R x: a
    feed-forward with routing of its own, written with torch operations."""

    def __init__(self, hidden_size: int, n_experts: int):
        self.hidden_size, self.n_experts = hidden_size, n_experts
        self.router = self.experts = None

    def param_specs(self):
        H = self.hidden_size
        specs = {"router.weight": ParamSpec((self.n_experts, H))}
        specs.update({f"expert.{e}.weight": ParamSpec((H, H)) for e in range(self.n_experts)})
        return specs

    def load(self, fetch):
        self.router = fetch("router.weight")
        self.experts = torch.stack([fetch(f"expert.{e}.weight") for e in range(self.n_experts)])

    def forward(self, x, ctx, residual):
        r = x.float() @ self.router.float().T
        best = r.argmax(-1)
        y = torch.bmm(self.experts[best].float(), x.float()[:, :, None])[:, :, 0] * torch.sigmoid(r.max(-1).values)[:, None]
        ops.residual_add(residual, y.to(x.dtype).contiguous())


def norm(H, eps, prefix):
    return PartSpec("rmsnorm", {"size": H, "eps": eps}, prefix=prefix)


def spec_of(H, V, layers, schedule=None, eps=1e-5):
    return ModelSpec(hidden_size=H, vocab_size=V,
                     embedding=PartSpec("token_embedding", {"vocab_size": V, "hidden_size": H}, prefix="emb."),
                     layers=layers, schedule=schedule or [ScheduleEntry(i) for i in range(len(layers))],
                     final_norm=norm(H, eps, "norm."), head=PartSpec("linear_head", {"vocab_size": V, "hidden_size": H}, prefix="head."),
                     max_positions=4096)


def layer(i, H, mixer, ffn, eps=1e-5):
    return LayerSpec("prenorm", f"l{i}.", {"norm1": norm(H, eps, "n1."), "mixer": mixer, "norm2": norm(H, eps, "n2."), "ffn": ffn})


def attention_spec(H, nh, nkv, hd, window=None, theta=1e4, bias=True, kind="rope_neox", rotary_dim=None):
    return PartSpec("paged_attention", {"hidden_size": H, "n_heads": nh, "n_kv_heads": nkv, "head_dim": hd, "bias": bias,
                                        "window": window, "position": PartSpec(kind, {"head_dim": hd, "theta": theta,
                                                                                      "rotary_dim": rotary_dim})}, prefix="attn.")


def build(spec, dtype, seed=0, std=0.05):
    model = Model(spec)
    src = RandomSource(seed, dtype, DEV, std)
    model.load(src, dtype, DEV)
    src_cpu = RandomSource(seed, dtype, "cpu", std)
    src_cpu.expect(model.named_params())
    weights = {n: src_cpu.tensor(n).double() for n in src_cpu.names()}
    return model, weights


def run_whole_and_cut(model, toks, block_size=8, num_pages=64):
    """logits of every position, once as one step and once in portions and single tokens"""
    runner = ModelRunner(model, block_size=block_size, num_pages=num_pages, max_seqs=4)
    reqs = {"a": toks}
    whole = ru.run_trace(runner, ru.trace_whole(reqs))
    cut = ru.run_trace(runner, ru.trace_mixed(reqs, seed=1, decode_tail=9))
    return (torch.stack([whole[("a", p)] for p in range(len(toks))]).double(),
            torch.stack([cut[("a", p)] for p in range(len(toks))]).double())


def agree(whole, cut, dtype):
    """float32: the same bits however the tokens were cut; bfloat16: few rows and many rows go
    through matrix kernels that sum in different orders"""
    if dtype == torch.float32:
        return torch.equal(whole, cut)
    return float((whole - cut).abs().max()) <= 2e-2 * float(whole.abs().max())


def head_of(w, h, eps=1e-5):
    return plain.rms_norm(h, w["norm.weight"], eps) @ w["head.weight"].T


TOKS = [(7 * i + 3) % 50 for i in range(45)]


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 3e-2)])
def test_embedding_norm_head_alone(dtype, tol):
    H, V = 40, 50
    model, w = build(spec_of(H, V, [layer(0, H, PartSpec("test_no_mixer"), PartSpec("test_no_ffn"))]), dtype)
    whole, cut = run_whole_and_cut(model, TOKS)
    want = head_of(w, w["emb.weight"][torch.tensor(TOKS)])
    assert float((whole - want).abs().max()) < tol * float(want.abs().max()) and agree(whole, cut, dtype)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 3e-2)])
@pytest.mark.parametrize("nh,nkv,hd,window,rot,kind", [(4, 2, 16, None, None, "rope_neox"), (3, 3, 32, 12, 16, "rope_neox"),
                                                        (2, 1, 48, 20, None, "rope_interleaved")])
def test_attention_mixer_alone(dtype, tol, nh, nkv, hd, window, rot, kind):
    """attention with q/k/v bias, full or partial rotary in either pairing, with and without a window"""
    H, V, theta, T = 40, 50, 5e3, len(TOKS)
    model, w = build(spec_of(H, V, [layer(0, H, attention_spec(H, nh, nkv, hd, window, theta, True, kind, rot),
                                          PartSpec("test_no_ffn"))]), dtype)
    whole, cut = run_whole_and_cut(model, TOKS, block_size=16)
    h = w["emb.weight"][torch.tensor(TOKS)]
    x = plain.rms_norm(h, w["l0.n1.weight"], 1e-5)
    proj = lambda n: x @ w[f"l0.attn.{n}_proj.weight"].T + w[f"l0.attn.{n}_proj.bias"]
    q, k, v = proj("q").reshape(T, nh, hd), proj("k").reshape(T, nkv, hd), proj("v").reshape(T, nkv, hd)
    r = rot or hd

    def rotate(t):
        out = t.clone()
        for p in range(T):
            if kind == "rope_neox":
                out[p, :, :r] = plain.rope_neox(t[p, :, :r], p, theta)
            else:
                for i in range(r // 2):
                    ang = p / (theta ** (2 * i / r))
                    a, b = t[p, :, 2 * i], t[p, :, 2 * i + 1]
                    out[p, :, 2 * i], out[p, :, 2 * i + 1] = a * math.cos(ang) - b * math.sin(ang), a * math.sin(ang) + b * math.cos(ang)
        return out

    att = plain.causal_attention(rotate(q), rotate(k), v, nh, nkv, window)
    want = head_of(w, h + att.reshape(T, nh * hd) @ w["l0.attn.o_proj.weight"].T)
    scale = float(want.abs().max())
    assert float((whole - want).abs().max()) < tol * scale
    assert float((cut - want).abs().max()) < tol * scale


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 3e-2)])
def test_feed_forwards_alone(dtype, tol):
    H, V = 40, 50
    dense = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": 56}, prefix="mlp.")
    moe = PartSpec("sparse_moe", {"hidden_size": H, "n_experts": 5, "top_k": 2, "expert_intermediate_size": 24,
                                  "norm_topk_prob": True, "shared_intermediate_size": 32}, prefix="moe.")
    model, w = build(spec_of(H, V, [layer(0, H, PartSpec("test_no_mixer"), dense), layer(1, H, PartSpec("test_no_mixer"), moe)]),
                     dtype, std=0.2)
    whole, cut = run_whole_and_cut(model, TOKS)
    h = w["emb.weight"][torch.tensor(TOKS)]
    x = plain.rms_norm(h, w["l0.n2.weight"], 1e-5)
    h = h + plain.swiglu_mlp(x, w["l0.mlp.gate_proj.weight"], w["l0.mlp.up_proj.weight"], w["l0.mlp.down_proj.weight"])
    x = plain.rms_norm(h, w["l1.n2.weight"], 1e-5)
    ex = [tuple(w[f"l1.moe.experts.{e}.{n}_proj.weight"] for n in ("gate", "up", "down")) for e in range(5)]
    sh = tuple(w[f"l1.moe.shared_expert.{n}_proj.weight"] for n in ("gate", "up", "down"))
    margins = []
    f = torch.stack([plain.moe_ffn_token(x[t], w["l1.moe.gate.weight"], ex, 2, True, sh, w["l1.moe.shared_expert_gate.weight"],
                                         margins) for t in range(len(TOKS))])
    want = head_of(w, h + f)
    keep = [t for t in range(len(TOKS)) if dtype == torch.float32 or margins[t] > 0.01]
    assert len(keep) > 0.8 * len(TOKS)
    assert float((whole - want)[keep].abs().max()) < tol * float(want.abs().max()) and agree(whole[keep], cut[keep], dtype)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 3e-2)])
def test_a_mixer_with_state_of_its_own(dtype, tol):
    """registered above, built from a spec and stepped; nothing in the package knows it"""
    H, V = 32, 50
    layers = [layer(0, H, PartSpec("test_running_mean", {"hidden_size": H}, prefix="rm."), PartSpec("test_no_ffn")),
              layer(1, H, attention_spec(H, 2, 2, 16), PartSpec("swiglu", {"hidden_size": H, "intermediate_size": 48}, prefix="mlp."))]
    model, w = build(spec_of(H, V, layers), dtype)
    assert model.cache_groups() == {("full",): None}
    runner = ModelRunner(model, block_size=8, num_pages=32, max_seqs=3)
    assert runner.storage.caches[0].state["sum"].shape == (3 + 1, H) and not runner.storage.caches[0].pages    # + the stand-in slot
    reqs = {"a": TOKS, "b": TOKS[5:30], "c": TOKS[::-1]}
    whole = ru.run_trace(runner, ru.trace_whole(reqs))
    mixed = ru.run_trace(runner, ru.trace_mixed(reqs, seed=4, max_live=3))       # slots are taken again, state starts at zero
    for key in whole:
        assert float((whole[key] - mixed[key]).abs().max()) <= tol * float(whole[key].abs().max())
    # against a plain computation of the first layer followed by the rest
    toks = reqs["a"]
    T = len(toks)
    h = w["emb.weight"][torch.tensor(toks)]
    x = plain.rms_norm(h, w["l0.n1.weight"], 1e-5)
    mean = torch.cumsum(x, 0) / torch.arange(1, T + 1, dtype=torch.float64)[:, None]
    h = h + mean @ w["l0.rm.mix.weight"].T
    x = plain.rms_norm(h, w["l1.n1.weight"], 1e-5)
    proj = lambda n: x @ w[f"l1.attn.{n}_proj.weight"].T + w[f"l1.attn.{n}_proj.bias"]
    q, k, v = (plain.rope_neox_rows(proj("q").reshape(T, 2, 16), range(T), 1e4),
               plain.rope_neox_rows(proj("k").reshape(T, 2, 16), range(T), 1e4), proj("v").reshape(T, 2, 16))
    h = h + plain.causal_attention(q, k, v, 2, 2, None).reshape(T, 32) @ w["l1.attn.o_proj.weight"].T
    x = plain.rms_norm(h, w["l1.n2.weight"], 1e-5)
    h = h + plain.swiglu_mlp(x, w["l1.mlp.gate_proj.weight"], w["l1.mlp.up_proj.weight"], w["l1.mlp.down_proj.weight"])
    want = head_of(w, h)
    got = torch.stack([whole[("a", p)] for p in range(T)]).double()
    assert float((got - want).abs().max()) < tol * float(want.abs().max())


def test_layer_order_is_data():
    """one layer run twice (with a cache of its own each time) and a layer that reads another's cache"""
    H, V, T = 32, 50, len(TOKS)
    att = lambda: attention_spec(H, 2, 1, 16, bias=False)
    layers = [layer(0, H, att(), PartSpec("test_no_ffn")), layer(1, H, att(), PartSpec("test_no_ffn"))]
    w_of = lambda w, l, n: w[f"l{l}.attn.{n}_proj.weight"]

    def attend(w, l, h, kv_from=None):
        x = plain.rms_norm(h, w[f"l{l}.n1.weight"], 1e-5)
        q = plain.rope_neox_rows((x @ w_of(w, l, "q").T).reshape(T, 2, 16), range(T), 1e4)
        if kv_from is None:
            k = plain.rope_neox_rows((x @ w_of(w, l, "k").T).reshape(T, 1, 16), range(T), 1e4)
            v = (x @ w_of(w, l, "v").T).reshape(T, 1, 16)
        else:
            k, v = kv_from
        return h + plain.causal_attention(q, k, v, 2, 1, None).reshape(T, 32) @ w_of(w, l, "o").T, (k, v)

    # layer 0 twice, then layer 1
    model, w = build(spec_of(H, V, layers, [ScheduleEntry(0), ScheduleEntry(0), ScheduleEntry(1)]), torch.float32)
    whole, cut = run_whole_and_cut(model, TOKS)
    h = w["emb.weight"][torch.tensor(TOKS)]
    for l in (0, 0, 1):
        h, _ = attend(w, l, h)
    want = head_of(w, h)
    assert float((whole - want).abs().max()) < 2e-5 * float(want.abs().max()) and torch.equal(whole, cut)
    # layer 1 reads the keys and values that layer 0 wrote
    model, w = build(spec_of(H, V, layers, [ScheduleEntry(0), ScheduleEntry(1, cache=0)]), torch.float32)
    whole, cut = run_whole_and_cut(model, TOKS)
    h = w["emb.weight"][torch.tensor(TOKS)]
    h, kv = attend(w, 0, h)
    h, _ = attend(w, 1, h, kv_from=kv)
    want = head_of(w, h)
    assert float((whole - want).abs().max()) < 2e-5 * float(want.abs().max()) and torch.equal(whole, cut)
    with pytest.raises(ValueError):
        Model(spec_of(H, V, layers, [ScheduleEntry(0, cache=1), ScheduleEntry(1)]))      # only an earlier entry's cache
    with pytest.raises(KeyError):
        Model(spec_of(H, V, [layer(0, H, PartSpec("no_such_mixer"), PartSpec("test_no_ffn"))]))


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 3e-2)])
def test_another_position_encoding_and_a_feed_forward_with_routing(dtype, tol):
    """both registered above from outside the package, with tensors of their own in the checkpoint;
    attention caches the keys as that encoding left them, so portions and single tokens must agree
    with whole prompts, and all with a plain computation"""
    H, V, nh, nkv, hd, E, T = 32, 50, 2, 1, 16, 3, len(TOKS)
    mixer = PartSpec("paged_attention", {"hidden_size": H, "n_heads": nh, "n_kv_heads": nkv, "head_dim": hd, "bias": False,
                                         "window": None, "position": PartSpec("test_decay_positions", {"head_dim": hd},
                                                                              prefix="pos.")}, prefix="attn.")
    ffn = PartSpec("test_top1_ffn", {"hidden_size": H, "n_experts": E}, prefix="route.")
    model, w = build(spec_of(H, V, [layer(0, H, mixer, ffn)]), dtype, std=0.2)
    assert {"l0.attn.pos.gain", "l0.route.router.weight", "l0.route.expert.2.weight"} <= set(model.named_params())
    whole, cut = run_whole_and_cut(model, TOKS)
    h = w["emb.weight"][torch.tensor(TOKS)]
    x = plain.rms_norm(h, w["l0.n1.weight"], 1e-5)
    f = DecayPositions.factors(w["l0.attn.pos.gain"], torch.arange(T)).double()
    q = (x @ w["l0.attn.q_proj.weight"].T).reshape(T, nh, hd) * f[:, None, :]
    k = (x @ w["l0.attn.k_proj.weight"].T).reshape(T, nkv, hd) / f[:, None, :]
    v = (x @ w["l0.attn.v_proj.weight"].T).reshape(T, nkv, hd)
    h = h + plain.causal_attention(q, k, v, nh, nkv, None).reshape(T, nh * hd) @ w["l0.attn.o_proj.weight"].T
    x = plain.rms_norm(h, w["l0.n2.weight"], 1e-5)
    r = x @ w["l0.route.router.weight"].T
    top2 = r.topk(2, -1).values
    y = torch.stack([torch.sigmoid(r[t].max()) * (w[f"l0.route.expert.{int(r[t].argmax())}.weight"] @ x[t]) for t in range(T)])
    want = head_of(w, h + y)
    keep = [t for t in range(T) if dtype == torch.float32 or float(top2[t, 0] - top2[t, 1]) > 0.05]     # clear choices
    assert len(keep) > 0.7 * T
    scale = float(want.abs().max())
    # (the two toy parts call library matrix products, whose rounding depends on the number of rows:
    # whole and cut agree within the tolerance, not bit for bit)
    assert float((whole - want)[keep].abs().max()) < tol * scale and float((cut - want)[keep].abs().max()) < tol * scale


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 3e-2)])
def test_a_recordable_mixer_with_a_cache_group_of_its_own(dtype, tol):
    """registered above from outside the package: it names its own cache group (pages that a window of its own
    ages), and its decode steps are recorded and replayed like the built-in attention's, with no change to the
    step function"""
    H, V, span, bs = 32, 50, 5, 4
    layers = [layer(0, H, PartSpec("test_window_mean", {"hidden_size": H, "span": span}, prefix="wm."), PartSpec("test_no_ffn")),
              layer(1, H, attention_spec(H, 2, 2, 16), PartSpec("swiglu", {"hidden_size": H, "intermediate_size": 48}, prefix="mlp."))]
    model, w = build(spec_of(H, V, layers), dtype)
    assert model.cache_groups() == {("test_window_mean", span): span, ("full",): None}
    # the mixer's own group gets few pages (a whole prompt of 45 tokens takes 12 of them for the length of its
    # step): they are given back as its window passes them, and taken again
    runner = ModelRunner(model, block_size=bs, num_pages={("full",): 40, ("test_window_mean", span): 13}, max_seqs=3)
    assert runner.use_graphs and runner.storage.caches[0].pages["x"].shape == (13 + 1, bs, H)      # + the stand-in page
    reqs = {"a": TOKS, "b": TOKS[5:30], "c": TOKS[::-1]}
    whole = ru.run_trace(runner, ru.trace_whole(reqs))
    steps = [{"entries": [{"id": r, "tokens": t[:6], "want": list(range(6))} for r, t in reqs.items()], "end": []}]
    for i in range(6, len(TOKS)):                                     # then all three decode in lockstep, recorded
        live = [r for r, t in reqs.items() if i < len(t)]
        steps.append({"entries": [{"id": r, "tokens": [reqs[r][i]], "want": [0]} for r in live],
                      "end": [r for r in live if i == len(reqs[r]) - 1]})
    decoded = ru.run_trace(runner, steps)
    assert {key[0] for key in runner._graphs} == {2, 3}, "the decode steps were not recorded"
    for key in whole:
        assert float((whole[key] - decoded[key]).abs().max()) <= tol * float(whole[key].abs().max()), key
    toks = reqs["a"]
    T = len(toks)
    h = w["emb.weight"][torch.tensor(toks)]
    x = plain.rms_norm(h, w["l0.n1.weight"], 1e-5)
    mean = torch.stack([x[max(0, t - span + 1):t + 1].mean(0) for t in range(T)])
    h = h + mean @ w["l0.wm.mix.weight"].T
    x = plain.rms_norm(h, w["l1.n1.weight"], 1e-5)
    proj = lambda n: x @ w[f"l1.attn.{n}_proj.weight"].T + w[f"l1.attn.{n}_proj.bias"]
    q, k, v = (plain.rope_neox_rows(proj("q").reshape(T, 2, 16), range(T), 1e4),
               plain.rope_neox_rows(proj("k").reshape(T, 2, 16), range(T), 1e4), proj("v").reshape(T, 2, 16))
    h = h + plain.causal_attention(q, k, v, 2, 2, None).reshape(T, 32) @ w["l1.attn.o_proj.weight"].T
    x = plain.rms_norm(h, w["l1.n2.weight"], 1e-5)
    h = h + plain.swiglu_mlp(x, w["l1.mlp.gate_proj.weight"], w["l1.mlp.up_proj.weight"], w["l1.mlp.down_proj.weight"])
    want = head_of(w, h)
    got = torch.stack([decoded[("a", p)] for p in range(T)]).double()
    assert float((got - want).abs().max()) < tol * float(want.abs().max())


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 3e-2)])
def test_a_rotary_with_a_table_of_frequency_factors(dtype, tol):
    """registered above from outside the package; the table reaches the rotating kernels (the one that rotates
    and writes the cache, and for few bfloat16 tokens the q/k/v product that does so in its epilogue)"""
    H, V, nh, nkv, hd, theta, T = 64, 50, 2, 1, 32, 300.0, len(TOKS)
    mixer = PartSpec("paged_attention", {"hidden_size": H, "n_heads": nh, "n_kv_heads": nkv, "head_dim": hd, "bias": True,
                                         "window": None, "position": PartSpec("test_banded_rope", {"head_dim": hd, "theta": theta},
                                                                              prefix="pos.")}, prefix="attn.")
    model, w = build(spec_of(H, V, [layer(0, H, mixer, PartSpec("test_no_ffn"))]), dtype, std=0.3)
    assert "l0.attn.pos.bands" in model.named_params()
    whole, cut = run_whole_and_cut(model, TOKS, block_size=16)
    h = w["emb.weight"][torch.tensor(TOKS)]
    x = plain.rms_norm(h, w["l0.n1.weight"], 1e-5)
    proj = lambda n: x @ w[f"l0.attn.{n}_proj.weight"].T + w[f"l0.attn.{n}_proj.bias"]
    factors = 1.0 + 8.0 * w["l0.attn.pos.bands"].abs()
    assert float(factors.max()) > 2.0

    def rotate(t):
        out = t.clone()
        for p in range(T):
            for i in range(hd // 2):
                ang = p / (theta ** (2 * i / hd)) / float(factors[i])
                a, b = t[p, :, i], t[p, :, i + hd // 2]
                out[p, :, i], out[p, :, i + hd // 2] = a * math.cos(ang) - b * math.sin(ang), a * math.sin(ang) + b * math.cos(ang)
        return out

    q, k, v = rotate(proj("q").reshape(T, nh, hd)), rotate(proj("k").reshape(T, nkv, hd)), proj("v").reshape(T, nkv, hd)
    want = head_of(w, h + plain.causal_attention(q, k, v, nh, nkv, None).reshape(T, nh * hd) @ w["l0.attn.o_proj.weight"].T)
    unbanded = head_of(w, h + plain.causal_attention(plain.rope_neox_rows(proj("q").reshape(T, nh, hd), range(T), theta),
                                                      plain.rope_neox_rows(proj("k").reshape(T, nkv, hd), range(T), theta),
                                                      v, nh, nkv, None).reshape(T, nh * hd) @ w["l0.attn.o_proj.weight"].T)
    scale = float(want.abs().max())
    assert float((unbanded - want).abs().max()) > 10 * tol * scale, "the factors make no difference in this test"
    assert float((whole - want).abs().max()) < tol * scale and float((cut - want).abs().max()) < tol * scale


# ---- blocks from outside the package that hand normed rows on to each other ------------------------------
from ferrox_amd.parts import BLOCKS, NORMS, Block  # noqa: E402


@BLOCKS.register("test_mixer_only")
class MixerOnly(Block):
    """h += mixer(norm1(h)), and nothing else.  It chains: it takes norm1(h) from the block before where that block
    has made it, and says what kind of rows its mixer accepts."""
    slots = {"norm1": NORMS, "mixer": MIXERS}
    chains_norms = True

    def __init__(self, parts, prefixes):
        self.norm1, self.mixer, self._prefixes = parts["norm1"], parts["mixer"], prefixes

    def children(self):
        return [(self._prefixes["norm1"], self.norm1), (self._prefixes["mixer"], self.mixer)]

    @property
    def first_norm(self):
        return self.norm1

    def takes_scale_later(self, act_dtype):
        return bool(self.mixer.takes_scale_later(act_dtype))

    def forward(self, h, ctx, cache, normed=None, then=None):
        if normed is not None:
            self.mixer.forward(normed, ctx, cache, h)
        elif not self.mixer.forward_from_residual(self.norm1, ctx, cache, h):
            self.mixer.forward(self.norm1.forward(h, ctx), ctx, cache, h)
        return None


@BLOCKS.register("test_ffn_only")
class FfnOnly(Block):
    """h += ffn(norm2(h)) around a mixer that does nothing.  It chains: a feed-forward that can norm the rows it
    has finished for the block that follows is told which norm that is, and what it leaves is handed on."""
    slots = {"mixer": MIXERS, "norm2": NORMS, "ffn": FEED_FORWARDS}
    chains_norms = True

    def __init__(self, parts, prefixes):
        self.mixer, self.norm2, self.ffn, self._prefixes = parts["mixer"], parts["norm2"], parts["ffn"], prefixes

    def children(self):
        return [(self._prefixes["norm2"], self.norm2), (self._prefixes["ffn"], self.ffn)]

    @property
    def first_norm(self):
        return self.norm2

    def forward(self, h, ctx, cache, normed=None, then=None):
        assert normed is None                       # (takes_scale_later is False and no block before it norms for it)
        ctx.carry = None
        more = {"then_norm": then} if then is not None and self.ffn.norms_after else {}
        if not self.ffn.forward_from_residual(self.norm2, ctx, h, **more):
            self.ffn.forward(self.norm2.forward(h, ctx), ctx, h, **more)
        out, ctx.carry = ctx.carry, None
        return out


@MIXERS.register("test_no_mixer_recordable")
class NoMixerRecordable(NoMixer):
    graph_safe = True


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "E"])
def test_two_chaining_blocks_from_outside_equal_the_built_in_block(model_folders, name, dtype):
    """Every layer of a model cut into two blocks defined here, one with the mixer and one with the feed-forward,
    which hand normed rows on through the blocks' optional protocol (`chains_norms`, `first_norm`,
    `takes_scale_later`, `forward(..., normed=, then=)`): the same kernels run in the same order as with the
    built-in pre-norm block, so the logits are the same bits, for whole prompts and for few tokens from recorded
    steps, where the feed-forward's last kernel norms for the next layer's mixer."""
    from conftest import TINY
    from ferrox_amd.config import Qwen2MoeConfig
    from ferrox_amd.engine.loading import load_model
    from ferrox_amd.models.qwen2_moe import build_spec
    from ferrox_amd.weights import Checkpoint
    folder = model_folders(name, "bfloat16" if name == "E" else dtype)
    built_in = load_model(folder, dtype, DEV)
    spec = build_spec(Qwen2MoeConfig.from_dict(TINY[name][0]), Checkpoint(folder).names())
    layers = []
    for ls in spec.layers:
        layers.append(LayerSpec("test_mixer_only", ls.prefix, {"norm1": ls.parts["norm1"], "mixer": ls.parts["mixer"]}))
        layers.append(LayerSpec("test_ffn_only", ls.prefix, {"mixer": PartSpec("test_no_mixer_recordable"),
                                                             "norm2": ls.parts["norm2"], "ffn": ls.parts["ffn"]}))
    spec.layers, spec.schedule = layers, [ScheduleEntry(i) for i in range(len(layers))]
    cut = Model(spec)
    cut.load(Checkpoint(folder), built_in.act_dtype, DEV)
    reqs = ru.make_requests(TINY[name][0]["vocab_size"], [40, 9, 70], 21)
    seen = []
    probe = ops.moe_combine

    def watching(*a, **kw):
        out = probe(*a, **kw)
        seen.append(out is not None)
        return out

    outs = []
    for model in (built_in, cut):
        runner = ModelRunner(model, block_size=64 if name == "E" else 16, num_pages=24, max_seqs=3)
        assert runner.use_graphs
        ops.moe_combine = watching
        try:
            outs.append((ru.run_trace(runner, ru.trace_whole(reqs)), ru.run_trace(runner, ru.trace_tail_decode(reqs, tail=6))))
        finally:
            ops.moe_combine = probe
        assert runner._graphs
        if dtype == "bfloat16":
            assert any(seen), "no feed-forward normed its rows for the layer after it: the chain was not exercised"
        seen.clear()
    for a, b in zip(outs[0], outs[1]):
        assert a.keys() == b.keys()
        for key in a:
            assert torch.equal(a[key], b[key]), f"{name} {dtype}: position {key} differs between the two ways of cutting a layer into blocks"
