"""An architecture that the package does not know, registered from here and taken through the front door:
a configuration class with key names of its own, a `build_spec` over the package's parts with tensor names of
its own, `register_architecture`, then `write_random_model`, `load_model`, `Engine(folder).generate`, the command
line and `trace_run`, against a plain forward pass written here.  Nothing in the package is changed for it.

The stand-in is no published model: dense layers only, adjacent-pair rotation over half of every head, no
biases, a norm over every head of q and of k before the rotation, a feed-forward gated by tanh-GELU, two stop
ids, and a head tied to an embedding table under another name.  What a configuration class must offer, and that `defaulted_keys` reaches the command line, is checked on
the way."""
import json
import math
import os
import subprocess
import sys
from dataclasses import dataclass, field

import pytest
import torch

import plain_qwen2moe as plain
import replay_util as ru
from conftest import ROOT

from ferrox_amd.config.base import ConfigError, ConfigReader
from ferrox_amd.models.registry import Architecture, architecture_of, known_architectures, register_architecture, resolve
from ferrox_amd.parts.base import LayerSpec, ModelSpec, PartSpec, ScheduleEntry


@dataclass(frozen=True)
class StandInConfig:
    n_vocab: int
    width: int
    depth: int
    heads: int
    kv_heads: int
    ff_width: int
    rope_base: float
    rope_fraction: float
    eps: float
    context: int
    stop_ids: tuple
    defaulted_keys: tuple = field(default=(), compare=False)

    @classmethod
    def from_dict(cls, raw, where="config.json"):
        r = ConfigReader(raw, where)
        cfg = cls(n_vocab=r.integer("n_vocab", minimum=1), width=r.integer("width", minimum=1), depth=r.integer("depth", minimum=1),
                  heads=r.integer("heads", minimum=1), kv_heads=r.integer("kv_heads", minimum=1),
                  ff_width=r.integer("ff_width", minimum=1), rope_base=r.number("rope_base", 10000.0, positive=True),
                  rope_fraction=r.number("rope_fraction", 1.0, positive=True), eps=r.number("eps", 1e-5, positive=True),
                  context=r.integer("context", 512, minimum=1), stop_ids=r.int_list("stop_ids", ()),
                  defaulted_keys=tuple(r.defaulted))
        if cfg.width % cfg.heads or cfg.heads % cfg.kv_heads:
            raise ConfigError(f"{where}: width {cfg.width}, heads {cfg.heads}, kv_heads {cfg.kv_heads} do not divide")
        return cfg

    def to_dict(self):
        d = {"architectures": ["StandInForCausalLM"], "model_type": "stand_in"}
        for k in ("n_vocab", "width", "depth", "heads", "kv_heads", "ff_width", "rope_base", "rope_fraction", "eps", "context"):
            d[k] = getattr(self, k)
        d["stop_ids"] = list(self.stop_ids)
        return d


def build_stand_in(cfg: StandInConfig, tensor_names=None) -> ModelSpec:
    hd = cfg.width // cfg.heads
    rot = int(hd * cfg.rope_fraction) // 2 * 2
    layers = []
    for l in range(cfg.depth):
        layers.append(LayerSpec("prenorm", f"blocks.{l}.", {
            "norm1": PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.eps}, prefix="ln_a."),
            "mixer": PartSpec("paged_attention", {
                "hidden_size": cfg.width, "n_heads": cfg.heads, "n_kv_heads": cfg.kv_heads, "head_dim": hd, "bias": False,
                "position": PartSpec("rope_interleaved", {"head_dim": hd, "theta": cfg.rope_base, "rotary_dim": rot}),
                "qk_norm": PartSpec("rmsnorm", {"size": hd, "eps": cfg.eps})},
                prefix="attn."),
            "norm2": PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.eps}, prefix="ln_f."),
            "ffn": PartSpec("gated_mlp", {"hidden_size": cfg.width, "intermediate_size": cfg.ff_width,
                                          "activation": "gelu_tanh"}, prefix="ff."),
        }))
    return ModelSpec(hidden_size=cfg.width, vocab_size=cfg.n_vocab,
                     embedding=PartSpec("token_embedding", {"vocab_size": cfg.n_vocab, "hidden_size": cfg.width}, prefix="wte."),
                     layers=layers, schedule=[ScheduleEntry(l) for l in range(cfg.depth)],
                     final_norm=PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.eps}, prefix="ln_out."),
                     head=PartSpec("linear_head", {"vocab_size": cfg.n_vocab, "hidden_size": cfg.width, "tied_to": "wte.weight"},
                                   prefix="unused_head."),
                     max_positions=cfg.context, eos_token_id=cfg.stop_ids or None)


RAW = {"architectures": ["StandInForCausalLM"], "model_type": "stand_in", "n_vocab": 211, "width": 96, "depth": 3,
       "heads": 6, "kv_heads": 2, "ff_width": 136, "rope_fraction": 0.5, "eps": 2e-6, "context": 300, "stop_ids": [3, 5]}


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def stand_in_forward(cfg: dict, w: dict, tokens) -> torch.Tensor:
    """the stand-in, whole sequence, float64, from the plain model's parts"""
    T, nh, nkv = len(tokens), cfg["heads"], cfg["kv_heads"]
    hd = cfg["width"] // nh
    rot = int(hd * cfg["rope_fraction"]) // 2 * 2
    theta, eps = cfg.get("rope_base", 10000.0), cfg["eps"]

    def rotate(x):                                            # adjacent pairs (2i, 2i+1) of the first `rot` dimensions
        out = x.clone()
        for t in range(T):
            for i in range(rot // 2):
                ang = plain.rope_angle(t, i, rot, theta, "float32")
                a, b = x[t, :, 2 * i], x[t, :, 2 * i + 1]
                out[t, :, 2 * i], out[t, :, 2 * i + 1] = a * math.cos(ang) - b * math.sin(ang), a * math.sin(ang) + b * math.cos(ang)
        return out

    h = w["wte.weight"][torch.tensor(tokens)]
    for l in range(cfg["depth"]):
        p = f"blocks.{l}."
        x = plain.rms_norm(h, w[p + "ln_a.weight"], eps)
        q = rotate(plain.rms_norm((x @ w[p + "attn.q_proj.weight"].T).reshape(T, nh, hd), w[p + "attn.q_norm.weight"], eps))
        k = rotate(plain.rms_norm((x @ w[p + "attn.k_proj.weight"].T).reshape(T, nkv, hd), w[p + "attn.k_norm.weight"], eps))
        v = (x @ w[p + "attn.v_proj.weight"].T).reshape(T, nkv, hd)
        h = h + plain.causal_attention(q, k, v, nh, nkv, None).reshape(T, nh * hd) @ w[p + "attn.o_proj.weight"].T
        x = plain.rms_norm(h, w[p + "ln_f.weight"], eps)
        h = h + (gelu_tanh(x @ w[p + "ff.gate_proj.weight"].T) * (x @ w[p + "ff.up_proj.weight"].T)) @ w[p + "ff.down_proj.weight"].T
    return plain.rms_norm(h, w["ln_out.weight"], eps) @ w["wte.weight"].T


def greedy(cfg, w, prompt, n, stop=()):
    toks, out = list(prompt), []
    for _ in range(n):
        t = int(torch.argmax(stand_in_forward(cfg, w, toks)[-1]))
        if t in stop:
            return out, "stop"
        out.append(t)
        toks.append(t)
    return out, "length"


@pytest.fixture(scope="module")
def stand_in():
    if "StandInForCausalLM" not in known_architectures():
        register_architecture(Architecture("StandInForCausalLM", "stand_in", StandInConfig, build_stand_in))
    return resolve(RAW)


def test_what_a_configuration_class_must_offer():
    class NoDict:
        @classmethod
        def from_dict(cls, raw, where=""):
            return cls()

    with pytest.raises(TypeError, match="to_dict"):
        register_architecture(Architecture("Broken", "broken", NoDict, build_stand_in))
    assert "Broken" not in known_architectures()


def test_registered_by_name_and_by_type(stand_in):
    assert stand_in.config_class is StandInConfig
    assert resolve({"model_type": "stand_in"}) is stand_in
    cfg = StandInConfig.from_dict(RAW)
    assert architecture_of(cfg) is stand_in
    assert cfg.defaulted_keys == ("rope_base",) and StandInConfig.from_dict(cfg.to_dict()) == cfg
    with pytest.raises(ConfigError, match="no registered architecture"):
        architecture_of(object())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_an_outside_architecture_through_the_front_door(stand_in, tmp_path, dtype):
    from ferrox_amd.engine.api import Engine
    from ferrox_amd.engine.loading import load_model, write_random_model
    from ferrox_amd.engine.runner import ModelRunner
    # logits are compared on weights of spread 0.05; generation on weights of spread 0.2, where the greedy
    # continuation depends on the whole model (under a tied head and small weights it repeats the last token)
    folder = str(tmp_path / "stand_in")
    write_random_model(dict(RAW), folder, seed=11, dtype=dtype, std=0.05 if dtype == "bfloat16" else 0.2, device="cuda:0")
    # norm weights are written as ones; give every norm weights of its own, so that a mix-up between them shows
    from safetensors.torch import load_file, save_file
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    g = torch.Generator().manual_seed(3)
    for name in sorted(tensors):
        if tensors[name].dim() == 1:
            tensors[name] = (1.0 + 0.3 * torch.randn(tensors[name].shape, generator=g)).to(tensors[name].dtype)
    assert sum(".q_norm." in n or ".k_norm." in n for n in tensors) == 2 * RAW["depth"]
    save_file(tensors, os.path.join(folder, "model.safetensors"))
    written = json.load(open(os.path.join(folder, "config.json")))
    assert written.pop("rope_base") == 10000.0              # (written in full; taken out again, so that reading defaults it)
    json.dump(written, open(os.path.join(folder, "config.json"), "w"))
    cfg, w = plain.load_folder(folder)
    assert cfg["architectures"] == ["StandInForCausalLM"] and "unused_head.weight" not in w and "wte.weight" in w
    model = load_model(folder, dtype, "cuda:0")
    assert model.head.weight.data_ptr() == model.embedding.weight.data_ptr()          # one table, tied by name
    assert isinstance(model.config, StandInConfig)
    # logits of every position, whole and cut into portions and single tokens (recorded decode steps)
    reqs = ru.make_requests(RAW["n_vocab"], [70, 33, 9], 17)
    runner = ModelRunner(model, block_size=16, num_pages=24, max_seqs=3)
    for what, steps in (("whole", ru.trace_whole(reqs)), ("mixed", ru.trace_mixed(reqs, seed=2, decode_tail=10))):
        got = ru.run_trace(runner, steps)
        for rid, toks in reqs.items():
            want = stand_in_forward(cfg, w, toks)
            mine = torch.stack([got[(rid, p)] for p in range(len(toks))]).double()
            err = float((mine - want).abs().max())
            bound = 2e-5 * float(want.abs().max()) if dtype == "float32" else 0.06 * float(want.std())
            assert err <= bound, f"{dtype} {what} {rid}: {err:.3e} > {bound:.3e}"
    assert runner._graphs
    if dtype != "float32":
        return
    # generation through the entry point, stop ids from this architecture's own key
    engine = Engine(folder, dtype="float32", block_size=16, num_pages=24, max_seqs=3)
    assert engine.eos_token_id == (3, 5) and engine.context_limit == 300
    prompts = [[7, 100, 42, 9], list(range(20, 60)), [200]]
    for p, c in zip(prompts, engine.generate_detailed(prompts, 10)):
        want, reason = greedy(cfg, w, p, 10, stop=(3, 5))
        assert (c.token_ids, c.finish_reason) == (want, reason)
        free, _ = greedy(cfg, w, p, 10)
        assert len(set(free)) >= 4, free
    # the command line and the replay program take the folder as they take any other
    cli = subprocess.run([sys.executable, "-c",
                          f"import sys; sys.path[:0] = [{ROOT!r}, {os.path.dirname(__file__)!r}]; import test_outside_architecture as t; "
                          f"t.register_architecture(t.Architecture('StandInForCausalLM', 'stand_in', t.StandInConfig, t.build_stand_in)); "
                          f"from ferrox_amd.cli import main; sys.exit(main(['-m', {folder!r}, '--tokens', '7,100,42,9', '-n', '10', "
                          f"'--temp', '0', '--repeat-penalty', '1', '--dtype', 'fp32', '--block-size', '16', '--ignore-eos']))"],
                         capture_output=True, text=True, timeout=600)
    assert cli.returncode == 0, cli.stderr[-2000:]
    assert [int(t) for t in cli.stdout.strip().split(",")] == greedy(cfg, w, prompts[0], 10)[0]
    assert "config keys defaulted: rope_base" in cli.stderr
    unknown = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "ferrox-amd"), "-m", folder, "--tokens", "7"],
                             capture_output=True, text=True, timeout=600)
    assert unknown.returncode == 2 and "StandInForCausalLM" in unknown.stderr          # a process that has not registered it
