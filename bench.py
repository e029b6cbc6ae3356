#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]          the one JSON line
    python bench.py --workload config3|config4|config5           serving runs through Engine.generate
    python bench.py --kernel-table decode_b1|decode_b8|decode_b16|..|decode_b64|prefill_128|prefill_512|prefill_2048|prefill_4096 [--out FILE]
                                                                 per-kernel times under rocprofv3 (a child process)

Model: the layer sizes of Qwen1.5-MoE-A2.7B with seeded random bf16 weights
N(0, 0.02) made on the GPU, seeded random token ids.  A "step" is one decode
step of the whole batch through the engine's own step function and sampling
kernel (greedy).  Default: batch 8, 2,048-token prompts prefilled through the
same step function, then W untimed and K timed decode steps (timed in three
consecutive parts, whose spread is reported beside the whole), driven as the
engine generates: the host a step ahead, a step launched with the ids of the
step before it still on the device, every id read by the host one step late.  The line also
carries: a 2,048-token prefill (one discarded run, median of five, every run a prompt of
its own, which moves the time by the experts its tokens choose); decode at
batch 1 and 64; the decode step's memory roofline for all three batch sizes:
bytes it has to read (every weight it uses once, the distinct experts counted
from the router's own choices in an untimed step, plus the cache of the live
requests) / time, against the published 8 TB/s; the ceilings measured on this
GPU by the simplest kernels (a streaming read, a copy, a loop of MFMA
products); and the same batch served through `Engine.generate` (scheduler,
sampling, ids read back), with the share of the time that the GPU waited for
the host; and 16 such prompts served in steps of at most 512 tokens, prompt
portions beside decoded tokens, launched kernel by kernel (`served_mixed`).
(The reference measures pp<N> / tg<N> the same way on synthetic ids with one
discarded warm-up and the median of three runs, ferrox-cli/src/bench_model.rs:35-60, 239-302.)
"""
from __future__ import annotations

import argparse
import json
import os
import random
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_HBM = 8.0e12          # bytes/s, MI355X HBM3E
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

from ferrox_amd.config import presets  # noqa: E402  (sizes are data: the config.json of each shape lies in the package)

A27B = presets.load("qwen1.5-moe-a2.7b")
FULL_LAYERS = A27B["num_hidden_layers"]
# the other shape of the family (not the default run): Qwen2-57B-A14B
A14B = presets.load("qwen2-57b-a14b")
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
    def prefill(self, T: int, reps: int = 5):
        """(median seconds, population standard deviation) of `reps` prefills of T tokens after one discarded run"""
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
        return statistics.median(times[1:]), statistics.pstdev(times[1:])

    def fill(self, ids, prompts, chunk: int = 2048):
        """Prefill the requests `ids` with `prompts` through the step function; returns their first sampled tokens."""
        from ferrox_amd import ops
        from ferrox_amd.engine.runner import StepEntry
        last = {}
        for rid, p in zip(ids, prompts):
            assert self.runner.admit(rid)
            for o in range(0, len(p), chunk):
                part = p[o:o + chunk]
                assert self.runner.reserve(rid, len(part))
                final = o + chunk >= len(p)
                lg = self.runner.step([StepEntry(rid, part, [len(part) - 1] if final else [])])
                if final:
                    last[rid] = int(ops.sample(lg)[0])
        return [last[r] for r in ids]

    def decode(self, batch: int, ctx: int, steps: int, warmup: int, parts: int = 3):
        """Prefill `batch` prompts of `ctx` tokens, then time `steps` decode steps, in `parts` consecutive parts.
        Returns (seconds per step over all steps, distinct experts per layer in a step, seconds per step of
        each part)."""
        torch = self.torch
        from ferrox_amd import debug, ops
        from ferrox_amd.engine.runner import StepEntry
        ids = [f"d{i}" for i in range(batch)]
        t0 = time.time()
        cur = self.fill(ids, self.prompts(batch, ctx))
        torch.cuda.synchronize()
        log(f"batch {batch}: prompts of {ctx} tokens prefilled in {time.time() - t0:.1f} s")

        pairs = [(i, i) for i in range(batch)]
        read = []                                  # every id that came back to the host, step by step

        def launch(known, on_device):
            """One decode step of all requests, launched: its tokens are `known`, or the ids `on_device` that the
            step before it sampled.  Returns (ids on the device, their copy in pinned memory, event after it)."""
            for rid in ids:
                assert self.runner.reserve(rid, 1)
            if on_device is None:
                lg = self.runner.step([StepEntry(rid, [t], [0]) for rid, t in zip(ids, known)])
            else:
                lg = self.runner.step([StepEntry(rid, [0], [0]) for rid in ids], feed=(on_device, pairs))
            out = ops.sample(lg)                   # greedy, on the device
            host = torch.empty(batch, dtype=torch.int32, pin_memory=True)
            host.copy_(out, non_blocking=True)
            copied = torch.cuda.Event()
            copied.record()
            return out, host, copied

        done_at = []                               # when the host saw each step's ids

        def collect(step):
            step[2].synchronize()
            done_at.append(time.perf_counter())
            read.append(step[1].tolist())

        # as the engine generates: the host is one step ahead; a step is launched with the ids of the step before
        # it still on the device, and those ids are read while it runs
        flying = launch(cur, None)
        for _ in range(warmup):
            nxt = launch(None, flying[0])
            collect(flying)
            flying = nxt
        parts = max(1, min(parts, steps))
        sizes = [steps // parts + (1 if i < steps % parts else 0) for i in range(parts)]
        torch.cuda.synchronize()
        collect(flying)                            # (it has ended; only its ids are read here)
        on_device, flying = flying[0], None
        first = len(done_at)
        t_all = time.perf_counter()
        for _ in range(steps):                     # exactly `steps` steps between the two synchronisations
            nxt = launch(None, on_device)
            if flying is not None:
                collect(flying)                    # (waits for the step before the one just launched)
            flying, on_device = nxt, nxt[0]
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t_all) / steps
        collect(flying)
        # a part's time per step, from when the host saw the last step before it end to when it saw its own last
        ends = [t_all] + done_at[first:]
        per_part, at = [], 0
        for n in sizes:
            per_part.append((ends[at + n] - ends[at]) / n)
            at += n
        assert all(0 <= t < self.cfg.vocab_size for row in read for t in row) and len(read) == warmup + steps + 1
        # one more, untimed, step that records which experts the router chose
        with debug.trace_routing() as trace:
            collect(launch(read[-1], None))
            per_layer = [len({e for tok in layer for e in tok}) for layer in trace.read()]
        distinct = sum(per_layer) / max(1, len(per_layer))
        for rid in ids:
            self.runner.release(rid)
        return dt, distinct, per_part

    def served_mixed(self, batch: int, ctx: int, new_tokens: int, portion: int = 512) -> dict:
        """`batch` prompts of `ctx` tokens behind `Engine.generate` with steps of at most `portion` tokens: every step
        but the last few carries the decoded tokens of the requests that are through their prompts beside a
        prompt portion of the next one, launched kernel by kernel (no step of this kind is recorded).  Beside the
        rate: the share of the time in which the GPU waited for the host between steps, and what the host spent
        launching against what the GPU spent running."""
        from ferrox_amd.engine.api import Engine
        per_seq = -(-(ctx + new_tokens + 1) // self.block_size)
        eng = Engine(model=self.model, block_size=self.block_size, num_pages=per_seq * batch + 8, max_seqs=batch,
                     max_tokens_per_step=portion, prefill_chunk=portion, ctx_size=ctx + new_tokens + 8)
        eng.time_steps = True
        prompts = self.prompts(batch, ctx)
        eng.generate(prompts[:2], max_new_tokens=4, ignore_eos=True)           # (kernels loaded, buffers there)
        self.torch.cuda.synchronize()
        t0 = time.perf_counter()
        out = eng.generate(prompts, max_new_tokens=new_tokens, ignore_eos=True)
        wall = time.perf_counter() - t0
        st = eng.last_stats
        assert all(len(o) == new_tokens for o in out)
        mixed = st["steps"] - st["decode_steps"]
        res = {"value": round(batch * (ctx + new_tokens) / wall, 1), "unit": "tokens/s, prompts and generation",
               "batch": batch, "prompt_tokens": ctx, "new_tokens": new_tokens, "portion": portion,
               "seconds": round(wall, 3), "steps": st["steps"], "steps_with_portions": mixed,
               "ms_per_step": round(1e3 * wall / st["steps"], 3),
               "host_share": round(1.0 - st["gpu_seconds"] / wall, 4),
               "host_launch_over_gpu": round(st["launch_seconds"] / st["gpu_seconds"], 3)}
        del eng
        return res

    def roofline(self, batch: int, kv_len: int, distinct: float, dt: float, ceilings: dict | None = None) -> dict:
        achieved = self.decode_bytes(batch, kv_len, distinct) / dt
        out = {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": PEAK_HBM / 1e9, "unit": "GB/s",
               "frac": round(achieved / PEAK_HBM, 4)}
        if ceilings and ceilings.get("hbm_read_GBs"):       # the faster of the two streaming reads (plain, non-temporal)
            best = max(ceilings["hbm_read_GBs"], ceilings.get("hbm_read_nt_GBs", 0.0))
            out["frac_of_measured_read"] = round(achieved / 1e9 / best, 4)
        return out

    def served(self, batch: int, ctx: int, new_tokens: int) -> dict:
        """The same model behind `Engine.generate`: `batch` prompts of `ctx` tokens arrive together, `new_tokens`
        greedy tokens each, through the scheduler (2,048-token portions), the sampling kernel and the read-back
        of the ids that the next step needs."""
        from ferrox_amd.engine.api import Engine
        per_seq = -(-(ctx + new_tokens + 1) // self.block_size)
        eng = Engine(model=self.model, block_size=self.block_size, num_pages=per_seq * batch + 8, max_seqs=batch,
                     max_tokens_per_step=4096, prefill_chunk=4096, ctx_size=ctx + new_tokens + 8)
        eng.time_steps = True
        prompts = self.prompts(batch, ctx)
        # once untimed: decode steps are recorded (a HIP graph per number of sequences and length bound) the first
        # time their shape occurs, which costs a few hundred ms that a serving process pays once
        eng.generate(prompts, max_new_tokens=new_tokens, ignore_eos=True)
        self.torch.cuda.synchronize()
        t0 = time.perf_counter()
        out = eng.generate(prompts, max_new_tokens=new_tokens, ignore_eos=True)
        wall = time.perf_counter() - t0
        st = eng.last_stats
        assert all(len(o) == new_tokens for o in out)
        n_dec = max(1, st["decode_steps"])
        dec_wall = st["decode_gpu_seconds"] + st["decode_gap_seconds"]
        res = {"value": round(batch * new_tokens / wall, 1), "unit": "generated tokens/s, prompts included",
               "batch": batch, "prompt_tokens": ctx, "new_tokens": new_tokens, "seconds": round(wall, 3),
               "steps": st["steps"], "decode_ms_per_step": round(1e3 * dec_wall / n_dec, 3),
               "decode_tokens_per_s": round(batch * n_dec / dec_wall, 1) if dec_wall > 0 else None,
               "host_share_decode": round(st["decode_gap_seconds"] / dec_wall, 4) if dec_wall > 0 else None,
               "host_share": round(1.0 - st["gpu_seconds"] / wall, 4)}
        del eng
        return res


def measure_ceilings(torch) -> dict:
    """What the simplest kernels reach on this GPU: streaming reads of 2 GiB (plain loads, and loads with the
    non-temporal hint that the engine's weight and cache streams use), a copy, a loop of bf16 MFMA products."""
    import ctypes
    from ferrox_amd.csrc.build import load_library
    lib = load_library("probe")
    vp, ci, cl = ctypes.c_void_p, ctypes.c_int, ctypes.c_long
    lib.fx_probe_read.argtypes, lib.fx_probe_copy.argtypes = [vp, vp, cl, vp, ci], [vp, vp, vp, cl]
    lib.fx_probe_mfma.argtypes = [vp, ci, ci, vp]
    stream = vp(torch.cuda.current_stream().cuda_stream)
    n = 1 << 31
    src = torch.empty(n, dtype=torch.uint8, device="cuda:0").random_(0, 255)
    dst = torch.empty(n, dtype=torch.uint8, device="cuda:0")
    out = torch.zeros(64, dtype=torch.float32, device="cuda:0")

    def timed(call, reps=5):
        call()
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(reps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            call()
            b.record()
            b.synchronize()
            best = min(best, a.elapsed_time(b) * 1e-3)
        return best

    def must(rc):
        if rc:
            raise RuntimeError(lib.fx_last_error().decode())

    t_read = timed(lambda: must(lib.fx_probe_read(stream, vp(src.data_ptr()), n, vp(out.data_ptr()), 0)))
    t_read_nt = timed(lambda: must(lib.fx_probe_read(stream, vp(src.data_ptr()), n, vp(out.data_ptr()), 1)))
    t_copy = timed(lambda: must(lib.fx_probe_copy(stream, vp(dst.data_ptr()), vp(src.data_ptr()), n)))
    blocks, iters = 256 * 8, 20000
    t_mfma = timed(lambda: must(lib.fx_probe_mfma(stream, blocks, iters, vp(out.data_ptr()))))
    flops = blocks * 4 * iters * 8 * 2 * 16 * 16 * 32
    del src, dst
    torch.cuda.empty_cache()
    return {"hbm_read_GBs": round(n / t_read / 1e9, 1), "hbm_read_nt_GBs": round(n / t_read_nt / 1e9, 1), "hbm_copy_GBs": round(2 * n / t_copy / 1e9, 1),
            "mfma_bf16_TFLOPs": round(flops / t_mfma / 1e12, 1)}


# ---- serving workloads (Engine.generate) ----------------------------------------------------------------------
WORKLOADS = {
    # name: (shape, config overrides, description)
    "config3": ("a2.7b", {}, "B=8 and B=64 requests, 2,048-token prompts, 256 new tokens"),
    "config4": ("57b-a14b", {}, "32 requests, prompts uniform in 512..16,384, 128 new tokens, 512-token portions"),
    "config5": ("57b-a14b", {"use_sliding_window": True, "sliding_window": 4096, "max_window_layers": 14},
                "8 requests of 24,576 tokens + 256 greedy tokens; then 64 requests at depths 1k..24k decoding; window 4096 on "
                "layers >= 14"),
}


def run_workload(name: str, args) -> int:
    import torch
    from ferrox_amd.engine.api import Engine
    from ferrox_amd.engine.loading import random_model
    shape_key, overrides, what = WORKLOADS[name]
    shape_name, shape = SHAPES[shape_key]
    cfg = dict(shape, **overrides)
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    rng = random.Random(4321)
    V = cfg["vocab_size"]
    t0 = time.time()
    model = random_model(cfg, seed=0, dtype=args.dtype, device="cuda:0")
    torch.cuda.synchronize()
    log(f"{name}: {shape_name}, {cfg['num_hidden_layers']} layers, made in {time.time() - t0:.1f} s; {what}")
    bs = args.block_size
    results = []

    def serve(prompts, new_tokens, chunk, budget, max_seqs, pages, label, warm=True):
        eng = Engine(model=model, block_size=bs, num_pages=pages, max_seqs=max_seqs, max_tokens_per_step=budget,
                     prefill_chunk=chunk, ctx_size=cfg["max_position_embeddings"])
        eng.time_steps = True
        if warm:                                   # record the decode graphs of this batch shape ahead of the timed run
            eng.generate([p[:max(2, min(len(p), 64))] for p in prompts], max_new_tokens=min(new_tokens, 4), ignore_eos=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        out = eng.generate(prompts, max_new_tokens=new_tokens, ignore_eos=True)
        wall = time.perf_counter() - t0
        st = eng.last_stats
        n_prompt, n_new = sum(len(p) for p in prompts), sum(len(o) for o in out)
        dec_wall = st["decode_gpu_seconds"] + st["decode_gap_seconds"]
        r = {"workload": name, "case": label, "requests": len(prompts), "prompt_tokens": n_prompt, "new_tokens": n_new,
             "seconds": round(wall, 3), "tokens_per_s_all": round((n_prompt + n_new) / wall, 1),
             "generated_tokens_per_s": round(n_new / wall, 1), "steps": st["steps"], "preemptions": st["preemptions"],
             "decode_only_steps": st["decode_steps"],
             "decode_ms_per_step": round(1e3 * dec_wall / max(1, st["decode_steps"]), 3),
             "host_share": round(1.0 - st["gpu_seconds"] / wall, 4),
             "host_share_decode": round(st["decode_gap_seconds"] / dec_wall, 4) if dec_wall > 0 else None}
        log(json.dumps(r))
        results.append(r)
        del eng
        torch.cuda.empty_cache()

    def prompts_of(lengths):
        return [[rng.randrange(V) for _ in range(n)] for n in lengths]

    def pages_for(lengths, new):
        groups = 2 if overrides.get("use_sliding_window") else 1
        return sum(-(-(n + new + 1) // bs) for n in lengths) + 8 * groups

    if name == "config3":
        for B in (8, 64):
            L = [2048] * B
            serve(prompts_of(L), 256, 4096, 4096, B, pages_for(L, 256), f"B={B}")
    elif name == "config4":
        L = [rng.randint(512, 16384) for _ in range(32)]
        serve(prompts_of(L), 128, 512, 512 + 32, 32, pages_for(L, 128), "32 requests, 512-token portions")
    else:
        L = [24576] * 8
        serve(prompts_of(L), 256, 4096, 4096, 8, pages_for(L, 256), "8 x 24,576-token prompts, 256 new tokens")
        L = [rng.randint(1024, 24576) for _ in range(64)]
        serve(prompts_of(L), 32, 4096, 4096 + 64, 64, pages_for(L, 32), "64 requests at depths 1k..24k, 32 new tokens")
    print(json.dumps({"workload": name, "model": shape_name, "layers": cfg["num_hidden_layers"], "dtype": args.dtype,
                      "results": results}), flush=True)
    return 0


# ---- per-kernel table (rocprofv3 around a child process) ----------------------------------------------------------
KERNEL_TABLES = {"decode_b1": ("decode", 1), "decode_b8": ("decode", 8), "decode_b16": ("decode", 16), "decode_b17": ("decode", 17), "decode_b24": ("decode", 24),
                 "decode_b32": ("decode", 32), "decode_b64": ("decode", 64), "decode_b96": ("decode", 96), "decode_b128": ("decode", 128),
                 "prefill_2048": ("prefill", 2048), "prefill_512": ("prefill", 512), "prefill_128": ("prefill", 128),
                 "prefill_4096": ("prefill", 4096)}


def profile_run(what: str, args) -> int:
    """The child of `--kernel-table`: runs the workload with its kernels launched one by one, and before every
    stage of the model an empty marker kernel whose grid size says which stage follows (ferrox_amd.debug.region)."""
    import ctypes
    import torch
    from ferrox_amd import debug, ops
    from ferrox_amd.csrc.build import load_library
    from ferrox_amd.engine.runner import StepEntry
    kind, n = KERNEL_TABLES[what]
    shape_name, shape = SHAPES[args.shape]
    steps = max(1, args.steps)
    b = Bench(args.layers or shape["num_hidden_layers"], args.dtype, args.block_size, n if kind == "decode" else 1,
              args.ctx if kind == "decode" else max(args.ctx, n), steps + 8, shape)      # a prompt has to fit the pool
    b.runner.use_graphs = False
    lib = load_library("probe")
    lib.fx_probe_mark.argtypes = [ctypes.c_void_p, ctypes.c_int]
    labels: list = []

    def sink(name):
        if name not in labels:
            labels.append(name)
        lib.fx_probe_mark(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream), labels.index(name))

    distinct = 0.0
    if kind == "decode":
        ids = [f"d{i}" for i in range(n)]
        cur = b.fill(ids, b.prompts(n, args.ctx))

        def one_step(toks):
            for rid in ids:
                assert b.runner.reserve(rid, 1)
            lg = b.runner.step([StepEntry(rid, [t], [0]) for rid, t in zip(ids, toks)])
            debug.region("sample")
            return ops.sample(lg).tolist()

        for _ in range(2):
            cur = one_step(cur)
        with debug.trace_routing() as trace:
            cur = one_step(cur)
            per_layer = [len({e for tok in layer for e in tok}) for layer in trace.read()]
        distinct = sum(per_layer) / max(1, len(per_layer))
        torch.cuda.synchronize()
        debug.region_sink = sink
        for _ in range(steps):
            cur = one_step(cur)
        sink("end")
        debug.region_sink = None
    else:
        used = []
        for i in range(steps + 1):
            toks = b.prompts(1, n)[0]
            assert b.runner.admit("p") and b.runner.reserve("p", n)
            if i == 1:
                torch.cuda.synchronize()
                debug.region_sink = sink
            if i == 0:
                # the untimed run also counts the experts that the prompt's tokens choose: with random weights the
                # tokens of one sequence look alike to the routers of the later layers, and far fewer experts than
                # the model has are in use (about 30 of 60 a layer for 2,048 tokens)
                with debug.trace_routing() as trace:
                    b.runner.step([StepEntry("p", toks, [n - 1])])
                    used = [len({e for tok in layer for e in tok}) for layer in trace.read()]
            else:
                b.runner.step([StepEntry("p", toks, [n - 1])])
            b.runner.release("p")
        distinct = sum(used) / max(1, len(used))
        sink("end")
        debug.region_sink = None
    torch.cuda.synchronize()
    ffn = next((blk.ffn for blk in b.model.blocks if hasattr(blk.ffn, "shared_pieces")), None)
    print("PROFILE_RUN " + json.dumps({"labels": labels, "steps": steps, "distinct_experts": distinct,
                                       "shared_as_pieces": bool(ffn is not None and ffn.shared_pieces and
                                                                (n <= 16 if kind == "decode" else n * shape["num_experts_per_tok"] <= 1024))}),
          flush=True)
    return 0


def stage_costs(c, kind: str, n: int, ctx: int, distinct: float, pieces: bool, es: int = 2) -> dict:
    """stage -> (bytes it has to read, flops it has to do) per step, from the configuration: every weight once,
    the cache of the live requests, activations of a prompt once in and once out."""
    H, hd, L = c.hidden_size, c.head_dim, c.num_hidden_layers
    qw, kvw = c.num_attention_heads * hd, c.num_key_value_heads * hd
    E, k, Im, Is, V = c.num_experts, c.num_experts_per_tok, c.moe_intermediate_size, c.shared_expert_intermediate_size, c.vocab_size
    T = n                                               # tokens in the step
    used = distinct if distinct > 0 else E               # experts whose weights the step reads (counted from the routers' choices)
    rows = 1 if kind == "prefill" else n                # rows that go through the head
    act = lambda cols: T * cols * es                    # one activation matrix
    w = lambda elems: elems * es
    attn_bytes = L * (n * ctx * 2 * kvw * es if kind == "decode" else 2 * T * kvw * es + 2 * T * qw * es)
    attn_flops = L * (4 * c.num_attention_heads * hd * (n * ctx if kind == "decode" else T * (T + 1) / 2))
    sh_up, sh_dn = 2 * Is * H, H * Is
    costs = {
        "embed": (T * H * (es + 4), 0),
        "norm": (L * 2 * T * H * (4 + es), 0),
        "qkv": (L * (w((qw + 2 * kvw) * H) + act(H) + act(qw + 2 * kvw)), L * 2 * T * (qw + 2 * kvw) * H),
        "rope + cache write": (L * 2 * act(qw + 2 * kvw), 0),
        "attention": (attn_bytes, attn_flops),
        "o_proj": (L * (w(H * qw) + act(qw) + 2 * T * H * 4), L * 2 * T * H * qw),
        "router": (L * (w((E + 1) * H) + T * H * 4), L * 2 * T * (E + 1) * H),
        "experts gate/up": (L * (w(used * 2 * Im * H + (sh_up if pieces else 0)) + act(H) + T * k * Im * es),
                            L * 2 * T * (k * 2 * Im * H + (sh_up if pieces else 0))),
        "experts down": (L * (w(used * H * Im + (sh_dn if pieces else 0)) + T * k * Im * es + T * k * H * 4),
                         L * 2 * T * (k * H * Im + (sh_dn if pieces else 0))),
        "shared expert": (L * (w(sh_up + sh_dn) + act(H) + 2 * act(Is) + T * H * 4), L * 2 * T * (sh_up + sh_dn)),
        "combine": (L * T * H * 4 * (k + 3), 0),
        "final norm": (rows * H * (4 + es), 0),
        "head": (w(V * H) + rows * V * 4, 2 * rows * V * H),
        "sample": (rows * V * 4, 0),
    }
    return costs


def kernel_table(what: str, args) -> int:
    import csv
    import glob
    import re
    import subprocess
    import tempfile
    from ferrox_amd.config import Qwen2MoeConfig
    kind, n = KERNEL_TABLES[what]
    shape_name, shape = SHAPES[args.shape]
    steps = args.steps if args.steps != 64 else (3 if kind == "prefill" else 8)
    tmp = tempfile.mkdtemp(prefix="ferrox_prof_", dir="/tmp")
    child = [sys.executable, os.path.abspath(__file__), "--profile-run", what, "--steps", str(steps), "--shape", args.shape,
             "--layers", str(args.layers), "--ctx", str(args.ctx), "--dtype", args.dtype, "--block-size", str(args.block_size)]
    cmd = ["rocprofv3", "--kernel-trace", "--output-format", "csv", "-d", tmp, "-o", "p", "--"] + child
    log("running: " + " ".join(cmd))
    proc = subprocess.run(cmd, cwd=tmp, env=dict(os.environ, TMPDIR=tmp), capture_output=True, text=True, timeout=1100)
    info = next((json.loads(l[len("PROFILE_RUN "):]) for l in proc.stdout.splitlines() if l.startswith("PROFILE_RUN ")), None)
    traces = glob.glob(os.path.join(tmp, "**", "*kernel_trace.csv"), recursive=True)
    if proc.returncode != 0 or info is None or not traces:
        print(f"bench.py: the profiled run failed (exit {proc.returncode})\n{proc.stdout[-2000:]}\n{proc.stderr[-3000:]}", flush=True)
        return 1
    with open(traces[0], newline="") as f:
        rows = list(csv.DictReader(f))
    col = lambda *words: next(c for c in rows[0] if all(wd in c.lower() for wd in words))
    c_name, c_start, c_end, c_disp = col("kernel", "name"), col("start"), col("end"), col("dispatch")
    c_grid, c_wg = col("grid", "x"), col("workgroup", "x")
    rows.sort(key=lambda r: int(r[c_disp]))
    labels = info["labels"]
    stage, per_stage, first, last = None, {}, None, None
    for r in rows:
        name = r[c_name]
        if "probe_mark_kernel" in name:
            stage = labels[int(r[c_grid]) // max(1, int(r[c_wg])) - 1]
            if first is None:
                first = int(r[c_start])
            if stage == "end":
                stage = None
            continue
        if stage is None:
            continue
        dur = int(r[c_end]) - int(r[c_start])
        last = int(r[c_end])
        short = re.sub(r"^void ", "", re.sub(r"\(.*$", "", name))
        st = per_stage.setdefault(stage, {"ns": 0, "kernels": {}})
        st["ns"] += dur
        k = st["kernels"].setdefault(short, [0, 0])
        k[0] += 1
        k[1] += dur
    cfg = dict(shape)
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    c = Qwen2MoeConfig.from_dict(cfg)
    costs = stage_costs(c, kind, n, args.ctx, info["distinct_experts"], info["shared_as_pieces"])
    total_ns = sum(st["ns"] for st in per_stage.values())
    span_ns = (last - first) if first is not None and last is not None else 0
    lines = [f"Per-stage kernel times: {shape_name}, {c.num_hidden_layers} layers, {args.dtype}, "
             + (f"decode, batch {n}, {args.ctx}-token prompts" if kind == "decode" else f"prefill of {n} tokens")
             + f", {info['steps']} steps, kernels launched one by one (no HIP graph)",
             "Command (from the repository root, on an MI355X):",
             f"  python3 bench.py --kernel-table {what}" + (f" --shape {args.shape}" if args.shape != "a2.7b" else "")
             + (f" --layers {args.layers}" if args.layers else "") + (f" --ctx {args.ctx}" if args.ctx != 2048 else ""),
             "  (it runs itself under `rocprofv3 --kernel-trace`; an empty marker kernel before every stage tells the stages apart;",
             "   bytes = weights the stage uses once + cache + activations, flops from the sizes; peaks 8 TB/s and 2.5 PFLOP/s;",
             f"   experts whose weights a step reads: {info['distinct_experts']:.1f} of {c.num_experts} a layer, counted from the routers' choices)",
             f"sum of kernel times {total_ns / info['steps'] / 1e3:.1f} us per step; from the first kernel to the last "
             f"{span_ns / info['steps'] / 1e3:.1f} us per step (the host launches one by one here)",
             "",
             f"{'stage':22s} {'us/step':>9s} {'%':>5s} {'GB/s':>8s} {'of 8TB/s':>8s} {'TFLOP/s':>8s} {'of 2.5PF':>8s}  kernels (launches per step x avg us)"]
    table = {}
    for stage, st in sorted(per_stage.items(), key=lambda kv: -kv[1]["ns"]):
        t = st["ns"] / info["steps"] * 1e-9
        by, fl = costs.get(stage, (0, 0))
        kern = "; ".join(f"{nm} {cnt / info['steps']:.0f} x {ns / cnt / 1e3:.1f}" for nm, (cnt, ns) in
                         sorted(st["kernels"].items(), key=lambda kv: -kv[1][1]))
        gbs, tfs = by / t / 1e9 if t > 0 else 0, fl / t / 1e12 if t > 0 else 0
        lines.append(f"{stage:22s} {t * 1e6:9.1f} {100 * st['ns'] / max(1, total_ns):5.1f} {gbs:8.0f} {gbs / 8000:8.3f} "
                     f"{tfs:8.1f} {tfs / 2500:8.3f}  {kern}")
        table[stage] = {"us": round(t * 1e6, 1), "GBs": round(gbs, 1), "TFLOPs": round(tfs, 2)}
    text = "\n".join(lines)
    print(text, flush=True)
    if args.out:
        with open(args.out, "w") as f:
            f.write(text + "\n")
    print(json.dumps({"kernel_table": what, "us_per_step": round(total_ns / info["steps"] / 1e3, 1), "stages": table}), flush=True)
    return 0


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
    ap.add_argument("--no-served", action="store_true", help="skip the run through Engine.generate")
    ap.add_argument("--no-ceilings", action="store_true", help="skip the measured ceilings")
    ap.add_argument("--only-prefill", action="store_true", help="run the 2,048-token prefill alone (for profiling); prints its own line")
    ap.add_argument("--no-graphs", action="store_true", help="launch every decode kernel from the host instead of replaying a HIP graph")
    ap.add_argument("--workload", choices=sorted(WORKLOADS), help="a serving run through Engine.generate instead of the default line")
    ap.add_argument("--kernel-table", metavar="WHAT", choices=sorted(KERNEL_TABLES),
                    help="per-kernel times of one workload, measured by rocprofv3 around a child process")
    ap.add_argument("--out", help="with --kernel-table: also write the table to this file")
    ap.add_argument("--profile-run", metavar="WHAT", choices=sorted(KERNEL_TABLES), help=argparse.SUPPRESS)
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported", flush=True)
        return 2
    if args.workload:
        return run_workload(args.workload, args)
    if args.kernel_table:
        return kernel_table(args.kernel_table, args)
    if args.profile_run:
        return profile_run(args.profile_run, args)

    new_tokens = args.steps + args.warmup + 2
    max_batch = 1 if args.only_prefill else max(args.batch, 1 if args.no_points else 64)
    shape_name, shape = SHAPES[args.shape]
    full_layers = shape["num_hidden_layers"]
    b = Bench(args.layers or full_layers, args.dtype, args.block_size, max_batch, args.ctx, max(new_tokens, 64), shape)
    c = b.cfg
    if args.no_graphs:
        b.runner.use_graphs = False

    if args.only_prefill:
        t, sd = b.prefill(2048, reps=max(1, args.steps))
        print(json.dumps({"prefill_tokens": 2048, "ms": round(t * 1e3, 3), "sigma_ms": round(sd * 1e3, 3),
                          "tokens_per_s": round(2048 / t, 1),
                          "frac": round(b.prefill_flops(2048) / t / PEAK_FLOPS[args.dtype], 4)}), flush=True)
        return 0

    import torch
    ceilings = None if args.no_ceilings else measure_ceilings(torch)
    if ceilings:
        log(f"measured ceilings: {ceilings}")
    dt, distinct, per_part = b.decode(args.batch, args.ctx, args.steps, args.warmup)
    tok_s = args.batch / dt
    kv_mid = args.ctx + args.warmup + args.steps // 2
    roof = b.roofline(args.batch, kv_mid, distinct, dt, ceilings)
    log(f"decode batch {args.batch}: {dt * 1e3:.3f} ms/step, {tok_s:.1f} tok/s, {distinct:.1f} experts/layer, "
        f"{roof['achieved']:.0f} GB/s; parts {[round(x * 1e3, 3) for x in per_part]} ms/step")
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
        "spread": {"parts": len(per_part), "median_ms": round(statistics.median(per_part) * 1e3, 4),
                   "sigma_ms": round(statistics.pstdev(per_part) * 1e3, 4)},
        "roofline": roof,
    }
    if ceilings:
        out["ceilings"] = ceilings
    if not args.no_prefill:
        T = 2048
        t, sd = b.prefill(T)
        fl = b.prefill_flops(T)
        out["prefill"] = {"value": round(T / t, 1), "tokens": T, "ms": round(t * 1e3, 3), "sigma_ms": round(sd * 1e3, 3),
                          "frac": round(fl / t / PEAK_FLOPS[args.dtype], 4)}
        if ceilings and args.dtype == "bf16":
            out["prefill"]["frac_of_measured_mfma"] = round(fl / t / 1e12 / ceilings["mfma_bf16_TFLOPs"], 4)
        log(f"prefill {T}: {t * 1e3:.2f} ms (sigma {sd * 1e3:.2f}), {T / t:.0f} tok/s, {fl / t / 1e12:.1f} TFLOP/s")
    if not args.no_points:
        pts = {}
        for bs_, st in ((1, min(args.steps, 64)), (64, min(args.steps, 32))):
            w = min(args.warmup, 4)
            d, dist, parts = b.decode(bs_, args.ctx, st, w)
            pts[f"decode_b{bs_}"] = round(bs_ / d, 2)
            out[f"roofline_b{bs_}"] = b.roofline(bs_, args.ctx + w + st // 2, dist, d, ceilings)
            log(f"decode batch {bs_}: {d * 1e3:.3f} ms/step, {bs_ / d:.1f} tok/s, {dist:.1f} experts/layer, "
                f"{out[f'roofline_b{bs_}']['achieved']:.0f} GB/s")
        out["points"] = pts
    if not args.no_served:
        out["served"] = b.served(args.batch, args.ctx, 64)
        log(f"served through Engine.generate: {out['served']}")
        out["served_mixed"] = b.served_mixed(16, args.ctx, 32)
        log(f"served in steps of 512 tokens, prompt portions beside decoded tokens: {out['served_mixed']}")
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
