#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Model: the layer sizes of Qwen1.5-MoE-A2.7B with seeded random bf16 weights
N(0, 0.02) made on the GPU, seeded random token ids.  A "step" is one decode
step of the whole batch through the engine's own step function and sampling
kernel (greedy).  Default: batch 8, 2,048-token prompts prefilled through the
same step function, then W untimed and K timed decode steps.  The one JSON line
also carries a 2,048-token prefill, decode at batch 1 and 64, and the decode
step's memory roofline: bytes it has to read (every weight it uses once, the
distinct experts counted from the router's own choices in an untimed step, plus
the cache of the live requests) / time, against 8 TB/s.
(The reference measures pp<N> / tg<N> the same way on synthetic ids with one
discarded warm-up, ferrox-cli/src/bench_model.rs:239-302.)
"""
from __future__ import annotations

import argparse
import json
import os
import random
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_HBM = 8.0e12          # bytes/s, MI355X HBM3E
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

A27B = {
    "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe", "hidden_act": "silu",
    "num_hidden_layers": 24, "hidden_size": 2048, "num_attention_heads": 16, "num_key_value_heads": 16,
    "num_experts": 60, "num_experts_per_tok": 4, "norm_topk_prob": False, "moe_intermediate_size": 1408,
    "shared_expert_intermediate_size": 5632, "intermediate_size": 5632, "decoder_sparse_step": 1,
    "mlp_only_layers": [], "vocab_size": 151936, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
    "max_position_embeddings": 8192, "use_sliding_window": False, "sliding_window": 32768,
    "max_window_layers": 21, "tie_word_embeddings": False, "qkv_bias": True,
}
FULL_LAYERS = 24
# the other shape of the family (not the default run): Qwen2-57B-A14B
A14B = dict(A27B, num_hidden_layers=28, hidden_size=3584, num_attention_heads=28, num_key_value_heads=4,
            num_experts=64, num_experts_per_tok=8, moe_intermediate_size=2560, shared_expert_intermediate_size=20480,
            intermediate_size=18944, max_position_embeddings=32768)
SHAPES = {"a2.7b": ("Qwen1.5-MoE-A2.7B shape", A27B), "57b-a14b": ("Qwen2-57B-A14B shape", A14B)}


def log(*a):
    print("[bench]", *a, file=sys.stderr, flush=True)


class Bench:
    def __init__(self, layers: int, dtype: str, block_size: int, max_batch: int, ctx: int, new_tokens: int,
                 shape: dict = A27B):
        import torch
        from ferrox_amd.engine.loading import random_model
        from ferrox_amd.engine.runner import ModelRunner
        self.torch = torch
        cfg = dict(shape)
        cfg["num_hidden_layers"] = layers
        t0 = time.time()
        self.model = random_model(cfg, seed=0, dtype=dtype, device="cuda:0")
        torch.cuda.synchronize()
        log(f"model of {layers} layers made in {time.time() - t0:.1f} s")
        self.cfg = self.model.config
        per_seq = -(-(ctx + new_tokens + 1) // block_size)
        self.runner = ModelRunner(self.model, block_size=block_size, num_pages=per_seq * max_batch + 8,
                                  max_seqs=max_batch)
        self.block_size, self.dtype = block_size, dtype
        self.rng = random.Random(1234)

    def prompts(self, batch: int, n: int):
        V = self.cfg.vocab_size
        return [[self.rng.randrange(V) for _ in range(n)] for _ in range(batch)]

    # -- bytes a decode step has to read ----------------------------------
    def decode_bytes(self, batch: int, kv_len: int, distinct_experts: float) -> float:
        c, es = self.cfg, 2 if self.dtype in ("bf16", "bfloat16") else 4
        H, hd = c.hidden_size, c.head_dim
        qw, kvw = c.num_attention_heads * hd, c.num_key_value_heads * hd
        per_layer = (qw + 2 * kvw) * H + (qw + 2 * kvw) + H * qw + 2 * H          # attention + norms
        per_layer += c.num_experts * H + H                                          # router, shared gate
        per_layer += 3 * c.shared_expert_intermediate_size * H                      # shared expert
        per_layer += distinct_experts * 3 * c.moe_intermediate_size * H             # routed experts in use
        weights = c.num_hidden_layers * per_layer + c.vocab_size * H + H + batch * H  # + head, final norm, embedding rows
        kv = c.num_hidden_layers * batch * kv_len * 2 * kvw
        return (weights + kv) * es

    def prefill_flops(self, T: int) -> float:
        c = self.cfg
        H, hd = c.hidden_size, c.head_dim
        qw, kvw = c.num_attention_heads * hd, c.num_key_value_heads * hd
        lin = (qw + 2 * kvw) * H + H * qw + c.num_experts * H
        lin += 3 * c.shared_expert_intermediate_size * H + c.num_experts_per_tok * 3 * c.moe_intermediate_size * H
        attn = 4 * c.num_attention_heads * hd * (T + 1) / 2                         # causal: QK^T and PV
        return c.num_hidden_layers * (2 * lin + attn) * T + 2 * c.vocab_size * H    # head on the last row only

    # -- measurements --------------------------------------------------------
    def prefill(self, T: int, reps: int = 3):
        torch = self.torch
        from ferrox_amd.engine.runner import StepEntry
        times = []
        for r in range(reps + 1):
            toks = self.prompts(1, T)[0]
            assert self.runner.admit("p") and self.runner.reserve("p", T)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            logits = self.runner.step([StepEntry("p", toks, [T - 1])])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
            self.runner.release("p")
            assert torch.isfinite(logits).all()
        t = sorted(times[1:])[len(times[1:]) // 2]      # one discarded warm-up, median of the rest
        return t

    def decode(self, batch: int, ctx: int, steps: int, warmup: int, chunk: int = 2048):
        """Prefill `batch` prompts of `ctx` tokens, then time `steps` decode steps. Returns
        (seconds per step, distinct experts per layer in a step)."""
        torch = self.torch
        from ferrox_amd import ops
        from ferrox_amd.engine.runner import StepEntry
        from ferrox_amd.parts.moe import SparseMoE
        ids = [f"d{i}" for i in range(batch)]
        prompts = self.prompts(batch, ctx)
        t0 = time.time()
        last = {}
        for rid, p in zip(ids, prompts):
            assert self.runner.admit(rid)
            for o in range(0, ctx, chunk):
                part = p[o:o + chunk]
                assert self.runner.reserve(rid, len(part))
                final = o + chunk >= ctx
                lg = self.runner.step([StepEntry(rid, part, [len(part) - 1] if final else [])])
                if final:
                    last[rid] = int(ops.sample(lg)[0])
        torch.cuda.synchronize()
        log(f"batch {batch}: prompts of {ctx} tokens prefilled in {time.time() - t0:.1f} s")
        cur = [last[r] for r in ids]

        def one_step(toks):
            for rid in ids:
                assert self.runner.reserve(rid, 1)
            lg = self.runner.step([StepEntry(rid, [t], [0]) for rid, t in zip(ids, toks)])
            return ops.sample(lg).tolist()          # greedy, on the device; ids come back to the host

        for _ in range(warmup):
            cur = one_step(cur)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            cur = one_step(cur)
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / steps
        # one more, untimed, step that records which experts the router chose
        SparseMoE.record = []
        graphs, self.runner.use_graphs = self.runner.use_graphs, False      # the hook needs the eager path
        one_step(cur)
        self.runner.use_graphs = graphs
        torch.cuda.synchronize()
        per_layer = [len(set(t.flatten().tolist())) for t in SparseMoE.record]
        SparseMoE.record = None
        distinct = sum(per_layer) / max(1, len(per_layer))
        for rid in ids:
            self.runner.release(rid)
        return dt, distinct


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--ctx", type=int, default=2048, help="prompt length of the decode runs")
    ap.add_argument("--shape", default="a2.7b", choices=sorted(SHAPES), help="layer sizes (the default run is a2.7b)")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the model has (both are reported); 0 = all")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--block-size", type=int, default=64)
    ap.add_argument("--no-points", action="store_true", help="skip the batch-1 and batch-64 decode runs")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--only-prefill", action="store_true", help="run the 2,048-token prefill alone (for profiling); prints its own line")
    ap.add_argument("--no-graphs", action="store_true", help="launch every decode kernel from the host instead of replaying a HIP graph")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported", flush=True)
        return 2

    new_tokens = args.steps + args.warmup + 2
    max_batch = 1 if args.only_prefill else max(args.batch, 1 if args.no_points else 64)
    shape_name, shape = SHAPES[args.shape]
    full_layers = shape["num_hidden_layers"]
    b = Bench(args.layers or full_layers, args.dtype, args.block_size, max_batch, args.ctx, max(new_tokens, 64), shape)
    c = b.cfg
    if args.no_graphs:
        b.runner.use_graphs = False

    if args.only_prefill:
        t = b.prefill(2048, reps=max(1, args.steps))
        print(json.dumps({"prefill_tokens": 2048, "ms": round(t * 1e3, 3), "tokens_per_s": round(2048 / t, 1),
                          "frac": round(b.prefill_flops(2048) / t / PEAK_FLOPS[args.dtype], 4)}), flush=True)
        return 0

    dt, distinct = b.decode(args.batch, args.ctx, args.steps, args.warmup)
    tok_s = args.batch / dt
    kv_mid = args.ctx + args.warmup + args.steps // 2
    achieved = b.decode_bytes(args.batch, kv_mid, distinct) / dt
    log(f"decode batch {args.batch}: {dt * 1e3:.3f} ms/step, {tok_s:.1f} tok/s, {distinct:.1f} experts/layer, "
        f"{achieved / 1e9:.0f} GB/s")
    out = {
        "metric": f"decode tok/s (batch {args.batch}, {args.ctx:,}-token prompts)", "value": round(tok_s, 2), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(dt * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic: seeded random token ids, seeded random N(0,0.02) weights",
        "config": {
            "model": shape_name, "layers": c.num_hidden_layers, "layers_of_model": full_layers,
            "hidden": c.hidden_size, "heads": c.num_attention_heads, "kv_heads": c.num_key_value_heads,
            "head_dim": c.head_dim, "experts": c.num_experts, "top_k": c.num_experts_per_tok,
            "moe_intermediate": c.moe_intermediate_size, "shared_intermediate": c.shared_expert_intermediate_size,
            "vocab": c.vocab_size, "global_batch": args.batch, "seq_len": args.ctx, "new_tokens": args.steps,
            "block_size": args.block_size, "parallelism": "single GPU",
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": PEAK_HBM / 1e9, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM, 4)},
    }
    if not args.no_prefill:
        T = 2048
        t = b.prefill(T)
        fl = b.prefill_flops(T)
        out["prefill"] = {"value": round(T / t, 1), "tokens": T, "ms": round(t * 1e3, 3),
                          "frac": round(fl / t / PEAK_FLOPS[args.dtype], 4)}
        log(f"prefill {T}: {t * 1e3:.2f} ms, {T / t:.0f} tok/s, {fl / t / 1e12:.1f} TFLOP/s")
    if not args.no_points:
        pts = {}
        for bs_, st in ((1, min(args.steps, 64)), (64, min(args.steps, 32))):
            d, _ = b.decode(bs_, args.ctx, st, min(args.warmup, 4))
            pts[f"decode_b{bs_}"] = round(bs_ / d, 2)
            log(f"decode batch {bs_}: {d * 1e3:.3f} ms/step, {bs_ / d:.1f} tok/s")
        out["points"] = pts
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
