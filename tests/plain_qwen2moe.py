"""Plain, slow Qwen2-MoE: whole sequences, no cache, one function per part.

This file is the oracle of the test-suite.  It shares no code with the
package under test: it reads the model folder with the `safetensors` library,
keeps every tensor as a CPU torch tensor and loops where a loop is the
clearest way to write the formula.  Each function cites the place in the
reference (paths relative to the reference's `crates/` folder) whose formula
it follows; conventions that the reference does not have (config.json keys for
the layer plan and the window) are marked "convention".

Arithmetic is done in `dtype` (float64 by default, so that the oracle's own
rounding is far below what the tests look for).

`stored`, where a function takes it, is a rounding applied to exactly those
tensors that an engine with activations of reduced precision has to store:
normed rows, q/k/v after the bias, q and k after the rotation, the softmax's
unnormalised probabilities, the attention output, silu(gate) * up.  With
`stored=to_bfloat16` the model shows how far rounding at those places alone
moves the logits, which is what the bfloat16 tests measure the engine against;
None (the default) rounds nothing.
"""
from __future__ import annotations

import json
import math
import os

import torch


def to_bfloat16(x: torch.Tensor) -> torch.Tensor:
    """round to bfloat16 (nearest even) and back"""
    return x.to(torch.bfloat16).to(x.dtype)


# --------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------
def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """y = x / sqrt(mean(x^2) + eps) * w   (ferrox-core/src/matmul.rs:62-69).

    eps stands inside the square root, the weight multiplies (no `1 + w`).
    """
    mean_sq = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    scale = 1.0 / torch.sqrt(mean_sq + eps)
    return x * scale * weight


def rope_angle(pos: int, i: int, dim: int, theta: float, angles: str = "exact") -> float:
    """The angle of pair i at position pos: pos / theta^(2i/dim) (ferrox-core/src/attention.rs:26-27).

    The reference works it out in float32: `freq = 1.0 / theta.powf(2i / dim)`, `angle = pos as f32 * freq`.
    angles="float32" does the same: the frequency rounded to float32, times the position in float32 (one rounded
    product); deep in a sequence that angle is off the exact one by up to half a unit in its last place, 1e-4 rad
    at position 2,000, which is part of what the reference computes.  (The frequency is rounded from its exact
    value here; the reference's is whatever its float32 `powf` returns, which may differ in the last bit.)
    angles="exact" keeps float64 throughout.
    """
    freq = 1.0 / (theta ** ((2 * i) / dim))
    if angles == "exact":
        return pos * freq
    assert angles == "float32", angles
    import numpy as np
    return float(np.float32(pos) * np.float32(freq))


def rope_neox(vec: torch.Tensor, pos: int, theta: float, angles: str = "exact") -> torch.Tensor:
    """Split-half rotary on one head vector (ferrox-core/src/attention.rs:20-32).

    Pair (i, i + half) is rotated by `rope_angle(pos, i, dim, theta, angles)`; sine and cosine of that angle
    are taken in float64.
    """
    dim = vec.shape[-1]
    half = dim // 2
    out = vec.clone()
    for i in range(half):
        angle = rope_angle(pos, i, dim, theta, angles)
        s, c = math.sin(angle), math.cos(angle)
        a, b = vec[..., i], vec[..., i + half]
        out[..., i] = a * c - b * s
        out[..., i + half] = a * s + b * c
    return out


def rope_neox_rows(x: torch.Tensor, positions, theta: float, angles: str = "exact") -> torch.Tensor:
    """`rope_neox` on x[T, n_heads, head_dim], row t at positions[t]
    (ferrox-models/src/decoder.rs:3489-3507: every q head and k head, full head_dim)."""
    out = torch.empty_like(x)
    for t in range(x.shape[0]):
        out[t] = rope_neox(x[t], int(positions[t]), theta, angles)
    return out


def causal_attention(q, k, v, n_heads: int, n_kv_heads: int, window: int | None,
                     scale: float | None = None, stored=None) -> torch.Tensor:
    """Causal grouped-query attention over one whole sequence.

    q[T, n_heads, hd], k/v[T, n_kv_heads, hd]; row t is the query at position t
    and sees keys 0..=t (ferrox-core/src/attention.rs:418-452).  Head h reads
    kv head h // (n_heads // n_kv_heads) (attention.rs:432-438); scale is
    1/sqrt(hd) (attention.rs:433).  With a window W only the last W positions,
    the query's own included, are visible: t - s < W (attention.rs:498-513).
    Softmax in one go with max subtraction (equal to the reference's online
    form, attention.rs:146-175).
    """
    T, _, hd = q.shape
    group = n_heads // n_kv_heads
    if scale is None:
        scale = 1.0 / math.sqrt(hd)
    out = torch.zeros_like(q)
    for t in range(T):
        start = 0 if window is None else max(0, t + 1 - window)
        for h in range(n_heads):
            kv_h = h // group
            keys = k[start:t + 1, kv_h]            # [S, hd]
            vals = v[start:t + 1, kv_h]
            s = (keys @ q[t, h]) * scale
            p = torch.exp(s - s.max())
            if stored is None:
                p = p / p.sum()
                out[t, h] = p @ vals
            else:                 # the probabilities are rounded for the product, their sum is not
                out[t, h] = (stored(p) @ vals) / p.sum()
    return out


def route_top_k(logits: torch.Tensor, k: int, norm_topk_prob: bool):
    """Softmax over all experts, then top-k of the probabilities, optional
    renormalisation of the k weights (ferrox-moe/src/lib.rs:333-355).

    Ties: higher probability first, then lower expert index (the rule of the
    reference's GPU router, ferrox-metal/src/gpu.rs:686-699; its CPU sort leaves
    ties open).  Returns (ids list, weights tensor[k]).
    """
    e = torch.exp(logits - logits.max())
    probs = e / e.sum()
    order = sorted(range(probs.shape[0]), key=lambda i: (-float(probs[i]), i))
    ids = order[:k]
    w = torch.stack([probs[i] for i in ids])
    if norm_topk_prob:
        w = w / w.sum()
    return ids, w


def silu(x: torch.Tensor) -> torch.Tensor:
    """x / (1 + exp(-x))   (ferrox-core/src/matmul.rs:268-270)."""
    return x / (1.0 + torch.exp(-x))


def swiglu_mlp(x, w_gate, w_up, w_down, stored=None) -> torch.Tensor:
    """down( silu(gate x) * (up x) )   (ferrox-moe/src/lib.rs:655-658,
    ferrox-core/src/matmul.rs:274-280).  Weights are [out, in]."""
    act = silu(x @ w_gate.T) * (x @ w_up.T)
    if stored is not None:
        act = stored(act)
    return act @ w_down.T


def router_margin(logits: torch.Tensor, k: int) -> float:
    """Relative gap between the k-th and the (k+1)-th probability: how far the choice of
    experts is from flipping (1.0 if all experts are chosen)."""
    p = torch.softmax(logits, 0).sort(descending=True).values
    if k >= p.shape[0]:
        return 1.0
    return float((p[k - 1] - p[k]) / p[k - 1])


def combine_expert_outputs(routed, shared, hidden_dim: int, dtype=torch.float64) -> torch.Tensor:
    """sum of weight * routed output in the given order, then the shared outputs
    (ferrox-moe/src/lib.rs:735-752).  `routed`: list of (vector, weight)."""
    out = torch.zeros(hidden_dim, dtype=dtype)
    for vec, weight in routed:
        out = out + vec * weight
    for vec in shared:
        out = out + vec
    return out


def moe_ffn_token(x, router_w, experts, k, norm_topk_prob, shared, shared_gate_w, margins=None, forced_ids=None,
                  chosen=None, probs_out=None, stored=None):
    """One token through the sparse block.

    Router logits r = router . x with no bias (ferrox-models/src/decoder.rs:2915),
    routed sum in selection order (ferrox-moe/src/lib.rs:735-745), then the
    shared expert scaled by sigmoid(shared_gate . x)
    (ferrox-models/src/decoder.rs:2660-2679).
    `experts` is a list of (gate, up, down); `shared` one such triple or None.
    `forced_ids` replaces the router's choice of experts (their weights are still the router's
    probabilities); `chosen`, a list, receives the ids used; `probs_out`, a list, the router's
    probabilities of all experts.
    """
    logits = router_w @ x
    if probs_out is not None:
        probs_out.append(torch.softmax(logits, 0).tolist())
    ids, w = route_top_k(logits, k, norm_topk_prob)
    if forced_ids is not None and list(forced_ids) != ids:
        ids = [int(e) for e in forced_ids]
        e_ = torch.exp(logits - logits.max())
        w = torch.stack([(e_ / e_.sum())[i] for i in ids])
        if norm_topk_prob:
            w = w / w.sum()
    if chosen is not None:
        chosen.append(list(ids))
    if margins is not None:
        margins.append(router_margin(logits, k))
    routed = [(swiglu_mlp(x, *experts[e], stored=stored), w[j]) for j, e in enumerate(ids)]
    shared_out = []
    if shared is not None:
        y = swiglu_mlp(x, *shared, stored=stored)
        if shared_gate_w is not None:
            z = (shared_gate_w.reshape(-1) * x).sum()
            y = y * (1.0 / (1.0 + torch.exp(-z)))
        shared_out.append(y)
    return combine_expert_outputs(routed, shared_out, x.shape[0], x.dtype)


# --------------------------------------------------------------------------
# layer plan (convention of the config.json format; the reference reads GGUF
# keys and has only "the first n layers are dense", ferrox-models/src/config.rs:247-249)
# --------------------------------------------------------------------------
def layer_is_sparse(cfg: dict, l: int) -> bool:
    step = cfg.get("decoder_sparse_step", 1)
    return (l not in cfg.get("mlp_only_layers", [])
            and cfg.get("num_experts", 0) > 0
            and (l + 1) % step == 0)


def layer_window(cfg: dict, l: int):
    if cfg.get("use_sliding_window", False) and l >= cfg.get("max_window_layers", 0):
        return int(cfg["sliding_window"])
    return None


def head_dim_of(cfg: dict) -> int:
    return cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_attention_heads"]


# --------------------------------------------------------------------------
# whole model
# --------------------------------------------------------------------------
def load_folder(folder: str, dtype=torch.float64):
    from safetensors import safe_open

    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    weights = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            weights[name] = f.get_tensor(name).to(dtype)
    return cfg, weights


def forward(cfg: dict, w: dict, tokens, dtype=torch.float64, start_pos: int = 0, margins=None, routing=None,
            chosen=None, router_probs=None, stored=None, angles: str = "float32") -> torch.Tensor:
    """Logits[T, V] of one whole sequence (ferrox-models/src/decoder.rs:3014-3678
    followed by the head on every row, decoder.rs:2952-2973).

    `start_pos` shifts every position (used by the shift-invariance test only).
    `margins`, a list of T floats if given, receives for every position the smallest
    `router_margin` over the sparse layers.  `routing[t][j]` forces the experts of position t in the
    j-th sparse layer; `chosen`, a list, receives the experts used in the same shape, and
    `router_probs`, a list, the router's probabilities of all experts as [position][sparse layer][expert].
    `stored`: see the head of this file.  `angles`: how the rotation's angles are worked out, see `rope_angle`;
    the default is the reference's float32 product.
    """
    keep = stored if stored is not None else (lambda t: t)
    T = len(tokens)
    n_sparse = 0
    if chosen is not None:
        chosen[:] = [[] for _ in range(T)]
    if margins is not None:
        margins[:] = [1.0] * T
    if router_probs is not None:
        router_probs[:] = [[] for _ in range(T)]
    nh = cfg["num_attention_heads"]
    nkv = cfg.get("num_key_value_heads", nh)
    hd = head_dim_of(cfg)
    eps = cfg.get("rms_norm_eps", 1e-6)
    theta = cfg.get("rope_theta", 10000.0)
    positions = [start_pos + t for t in range(T)]

    h = w["model.embed_tokens.weight"][torch.tensor(tokens, dtype=torch.long)].to(dtype)  # no scale: decoder.rs:1279-1284
    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}."
        x = keep(rms_norm(h, w[p + "input_layernorm.weight"], eps))                 # decoder.rs:3225-3228
        q = x @ w[p + "self_attn.q_proj.weight"].T
        k = x @ w[p + "self_attn.k_proj.weight"].T
        v = x @ w[p + "self_attn.v_proj.weight"].T
        if p + "self_attn.q_proj.bias" in w:                                         # bias after the product,
            q = q + w[p + "self_attn.q_proj.bias"]                                   # before rotation:
            k = k + w[p + "self_attn.k_proj.bias"]                                   # decoder.rs:3234-3254
            v = v + w[p + "self_attn.v_proj.bias"]
        q, k, v = keep(q), keep(k), keep(v)
        q = keep(rope_neox_rows(q.reshape(T, nh, hd), positions, theta, angles))
        k = keep(rope_neox_rows(k.reshape(T, nkv, hd), positions, theta, angles))
        v = v.reshape(T, nkv, hd)                                                    # v is not rotated
        a = keep(causal_attention(q, k, v, nh, nkv, layer_window(cfg, l), stored=stored))
        h = h + a.reshape(T, nh * hd) @ w[p + "self_attn.o_proj.weight"].T          # no bias: decoder.rs:3549-3560
        x2 = keep(rms_norm(h, w[p + "post_attention_layernorm.weight"], eps))       # decoder.rs:3563-3566
        if layer_is_sparse(cfg, l):
            E = cfg["num_experts"]
            experts = [(w[p + f"mlp.experts.{e}.gate_proj.weight"],
                        w[p + f"mlp.experts.{e}.up_proj.weight"],
                        w[p + f"mlp.experts.{e}.down_proj.weight"]) for e in range(E)]
            shared = None
            gate_w = None
            if cfg.get("shared_expert_intermediate_size", 0) > 0:
                shared = (w[p + "mlp.shared_expert.gate_proj.weight"],
                          w[p + "mlp.shared_expert.up_proj.weight"],
                          w[p + "mlp.shared_expert.down_proj.weight"])
                gate_w = w[p + "mlp.shared_expert_gate.weight"]
            layer_margins = [] if margins is not None else None
            layer_chosen = []
            layer_probs = [] if router_probs is not None else None
            f = torch.stack([
                moe_ffn_token(x2[t], w[p + "mlp.gate.weight"], experts,
                              cfg["num_experts_per_tok"], cfg.get("norm_topk_prob", False),
                              shared, gate_w, layer_margins,
                              routing[t][n_sparse] if routing is not None else None, layer_chosen, layer_probs,
                              stored)
                for t in range(T)])
            if chosen is not None:
                for t in range(T):
                    chosen[t].append(layer_chosen[t])
            if router_probs is not None:
                for t in range(T):
                    router_probs[t].append(layer_probs[t])
            n_sparse += 1
            if margins is not None:
                for t in range(T):
                    margins[t] = min(margins[t], layer_margins[t])
        else:                                                                        # dense layer: decoder.rs:2902-2913
            f = swiglu_mlp(x2, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                           w[p + "mlp.down_proj.weight"], stored)
        h = h + f
    x = keep(rms_norm(h, w["model.norm.weight"], eps))                               # decoder.rs:3674-3677
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) \
        else w["lm_head.weight"]                                                     # loader.rs:1433-1436
    return x @ head.T


# --------------------------------------------------------------------------
# sampling (ferrox-models/src/sampling.rs)
# --------------------------------------------------------------------------
class XorShift64:
    """sampling.rs:66-84: shifts 13, 7, 17; seed 0 is replaced."""
    MASK = (1 << 64) - 1

    def __init__(self, seed: int):
        self.state = 0x9E3779B97F4A7C15 if seed == 0 else (seed & self.MASK)

    def next_u64(self) -> int:
        s = self.state
        s ^= (s << 13) & self.MASK
        s ^= s >> 7
        s ^= (s << 17) & self.MASK
        self.state = s
        return s

    def next_f32(self) -> float:
        return (self.next_u64() >> 40) / float(1 << 24)


def argmax_first(scores) -> int:
    """Greedy pick; on an exact tie the lowest index (a deliberate difference:
    the reference's `max_by` keeps the last maximum, sampling.rs:217-224)."""
    best, bi = None, 0
    for i, s in enumerate(scores):
        if best is None or s > best:
            best, bi = s, i
    return bi


def apply_history_penalties(scores: list, history, repetition_penalty=1.0,
                            presence_penalty=0.0, frequency_penalty=0.0):
    """sampling.rs:191-215.  The repetition penalty is applied once per
    occurrence in the history, as the reference's loop does."""
    if repetition_penalty != 1.0:
        for tok in history:
            if 0 <= tok < len(scores):
                s = scores[tok]
                scores[tok] = s / repetition_penalty if s > 0.0 else s * repetition_penalty
    if presence_penalty != 0.0 or frequency_penalty != 0.0:
        counts = {}
        for tok in history:
            counts[tok] = counts.get(tok, 0) + 1
        for tok, c in counts.items():
            if 0 <= tok < len(scores):
                scores[tok] -= frequency_penalty * c
                scores[tok] -= presence_penalty
    return scores


def sample(logits, rng: XorShift64, temperature=0.0, top_k=0, top_p=1.0,
           repetition_penalty=1.0, presence_penalty=0.0, frequency_penalty=0.0, history=()):
    """sampling.rs:93-189 in float64: penalties, greedy if temperature <= 0,
    else divide by temperature, softmax, top-k, top-p, renormalise, inverse-CDF walk."""
    scores = [float(x) for x in logits]
    apply_history_penalties(scores, history, repetition_penalty, presence_penalty, frequency_penalty)
    if temperature <= 0.0:
        return argmax_first(scores)
    scores = [s / temperature for s in scores]
    m = max(scores)
    exps = [math.exp(s - m) for s in scores]
    tot = sum(exps)
    probs = [e / tot for e in exps]
    order = sorted(range(len(probs)), key=lambda i: (-probs[i], i))
    if 0 < top_k < len(probs):
        for i in order[top_k:]:
            probs[i] = 0.0
    if top_p < 1.0:
        cum, cutoff = 0.0, len(order)
        for rank, i in enumerate(order):
            cum += probs[i]
            if cum >= top_p:
                cutoff = rank + 1
                break
        for i in order[cutoff:]:
            probs[i] = 0.0
    total = sum(probs)
    if total <= 0.0:
        return argmax_first([float(x) for x in logits])
    probs = [p / total for p in probs]
    draw = rng.next_f32()
    cum = 0.0
    for i, p in enumerate(probs):
        cum += p
        if draw < cum:
            return i
    for i in range(len(probs) - 1, -1, -1):
        if probs[i] > 0.0:
            return i
    return 0


def greedy_generate(cfg, w, prompt, n_new, dtype=torch.float64):
    """Prefill the prompt, then sample -> append -> forward, n_new times
    (ferrox-cli/src/run.rs:651-676), recomputing the whole sequence each time."""
    toks = list(prompt)
    out = []
    for _ in range(n_new):
        logits = forward(cfg, w, toks, dtype)[-1]
        nxt = int(torch.argmax(logits))
        out.append(nxt)
        toks.append(nxt)
    return out
