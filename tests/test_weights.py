"""The safetensors reader and writer, the by-name loader and its one error, random weights."""
import json
import os
import struct

import pytest
import torch

from conftest import TINY_A, TINY_B
from ferrox_amd.engine.loading import write_random_model
from ferrox_amd.engine.model import Model
from ferrox_amd.config import Qwen2MoeConfig
from ferrox_amd.models.qwen2_moe import build_spec
from ferrox_amd.parts.base import ParamSpec
from ferrox_amd.weights import (Checkpoint, CheckpointError, RandomSource, SafetensorsError, SafetensorsFile,
                                check_names, random_tensor, resident_dtype, write_safetensors)


def raw_file(path, header: dict, payload: bytes):
    blob = json.dumps(header).encode()
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)) + blob + payload)


def test_round_trip_and_other_readers_agree(tmp_path):
    ts = {"a": torch.randn(3, 4), "b": torch.randn(5).bfloat16(), "c": torch.arange(6, dtype=torch.int32).reshape(2, 3),
          "h": torch.randn(2, 2).half(), "empty": torch.zeros(0, 4)}
    p = str(tmp_path / "model.safetensors")
    write_safetensors(p, ts, {"who": "test"})
    f = SafetensorsFile(p)
    assert f.metadata == {"who": "test"} and set(f.names()) == set(ts)
    for n, t in ts.items():
        assert torch.equal(f.tensor(n), t) and f.info(n) == (t.dtype, tuple(t.shape))
    from safetensors import safe_open
    with safe_open(p, "pt") as g:
        for n, t in ts.items():
            assert torch.equal(g.get_tensor(n), t)


def test_malformed_files_are_refused(tmp_path):
    """The reference reader's rules (ferrox-safetensors/src/lib.rs:168-243, tests 400-588)."""
    p = str(tmp_path / "x.safetensors")
    ok = {"t": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}}
    raw_file(p, ok, b"\0" * 8)
    assert SafetensorsFile(p).info("t") == (torch.float32, (2,))
    cases = {
        "gap": ({"t": {"dtype": "F32", "shape": [2], "data_offsets": [4, 12]}}, b"\0" * 12, "contiguous"),
        "size": ({"t": {"dtype": "F32", "shape": [3], "data_offsets": [0, 8]}}, b"\0" * 8, "needs 12"),
        "trailing": (ok, b"\0" * 9, "data ends"),
        "dtype": ({"t": {"dtype": "F8_E4M3", "shape": [8], "data_offsets": [0, 8]}}, b"\0" * 8, "unsupported dtype"),
        "short": (ok, b"\0" * 4, "data ends"),
    }
    for name, (hdr, payload, word) in cases.items():
        raw_file(p, hdr, payload)
        with pytest.raises(SafetensorsError) as e:
            SafetensorsFile(p)
        assert word in str(e.value), name
    with open(p, "wb") as f:
        f.write(b"\1\2\3")
    with pytest.raises(SafetensorsError):
        SafetensorsFile(p)
    with open(p, "wb") as f:
        f.write(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(SafetensorsError):
        SafetensorsFile(p)


def test_sharded_index(tmp_path):
    write_safetensors(str(tmp_path / "s1.safetensors"), {"a": torch.ones(2)})
    write_safetensors(str(tmp_path / "s2.safetensors"), {"b": torch.zeros(3)})
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"a": "s1.safetensors", "b": "s2.safetensors"}}))
    c = Checkpoint(str(tmp_path))
    assert sorted(c.names()) == ["a", "b"] and torch.equal(c.tensor("b"), torch.zeros(3))
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"a": "s1.safetensors", "z": "s2.safetensors"}}))
    with pytest.raises(SafetensorsError):
        Checkpoint(str(tmp_path))
    with pytest.raises(SafetensorsError):
        Checkpoint(str(tmp_path / "missing"))


def test_names_are_those_of_the_checkpoint_format():
    names = set(Model(build_spec(Qwen2MoeConfig.from_dict(TINY_B))).named_params())
    want = {"model.embed_tokens.weight", "model.norm.weight"}
    for l in range(3):
        p = f"model.layers.{l}."
        want |= {p + "input_layernorm.weight", p + "post_attention_layernorm.weight", p + "self_attn.o_proj.weight"}
        want |= {p + f"self_attn.{x}_proj.{y}" for x in "qkv" for y in ("weight", "bias")}
    for l in (0, 2):
        want |= {f"model.layers.{l}.mlp.{x}_proj.weight" for x in ("gate", "up", "down")}
    p = "model.layers.1.mlp."
    want |= {p + "gate.weight", p + "shared_expert_gate.weight"}
    want |= {p + f"shared_expert.{x}_proj.weight" for x in ("gate", "up", "down")}
    want |= {p + f"experts.{e}.{x}_proj.weight" for e in range(6) for x in ("gate", "up", "down")}
    assert names == want                              # tied: no lm_head.weight
    assert "lm_head.weight" in Model(build_spec(Qwen2MoeConfig.from_dict(TINY_A))).named_params()
    shapes = Model(build_spec(Qwen2MoeConfig.from_dict(TINY_B))).named_params()
    assert shapes["model.layers.1.mlp.shared_expert_gate.weight"].shape == (1, 96)
    assert shapes["model.layers.1.mlp.experts.5.down_proj.weight"].shape == (96, 48)
    assert shapes["model.layers.2.self_attn.k_proj.weight"].shape == (32, 96)


def test_one_error_lists_everything_that_does_not_fit(tmp_path):
    folder = str(tmp_path / "m")
    write_random_model(dict(TINY_A), folder, 0, "float32")
    ck = Checkpoint(folder)
    model = Model(build_spec(Qwen2MoeConfig.from_dict(TINY_A), ck.names()))
    check_names(model.named_params(), ck)                       # fits
    tensors = {n: ck.tensor(n).clone() for n in ck.names()}
    del tensors["model.norm.weight"], tensors["model.layers.1.mlp.experts.3.up_proj.weight"]
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    tensors["lm_head.weight"] = torch.zeros(255, 64)
    tensors["model.layers.0.mlp.gate.weight"] = torch.zeros(8, 64, dtype=torch.int32)
    bad = str(tmp_path / "bad")
    os.makedirs(bad)
    write_safetensors(bad + "/model.safetensors", tensors)
    with pytest.raises(CheckpointError) as e:
        check_names(model.named_params(), Checkpoint(bad), bad)
    err, msg = e.value, str(e.value)
    assert err.missing == ["model.layers.1.mlp.experts.3.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert err.wrong_shape == [("lm_head.weight", (255, 64), (256, 64))]
    assert err.wrong_dtype[0][0] == "model.layers.0.mlp.gate.weight"
    for word in ("model.norm.weight", "rotary_emb.inv_freq", "[255, 64]", "[256, 64]", "missing", "unexpected"):
        assert word in msg


def test_tensors_nobody_asked_for_are_a_warning(tmp_path):
    """A file that holds more than the model wants still loads (the reference fetches by name and never looks at
    the rest, ferrox-models/src/loader.rs:564-629); one warning lists what is left over."""
    import warnings
    from ferrox_amd.weights import UnexpectedTensorsWarning
    folder = str(tmp_path / "m")
    write_random_model(dict(TINY_A), folder, 0, "float32")
    ck = Checkpoint(folder)
    model = Model(build_spec(Qwen2MoeConfig.from_dict(TINY_A), ck.names()))
    tensors = {n: ck.tensor(n).clone() for n in ck.names()}
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    tensors["model.layers.1.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    more = str(tmp_path / "more")
    os.makedirs(more)
    write_safetensors(more + "/model.safetensors", tensors)
    with warnings.catch_warnings(record=True) as caught:
        warnings.simplefilter("always")
        left = check_names(model.named_params(), Checkpoint(more), more)
    assert left == ["model.layers.0.self_attn.rotary_emb.inv_freq", "model.layers.1.self_attn.rotary_emb.inv_freq"]
    mine = [w for w in caught if issubclass(w.category, UnexpectedTensorsWarning)]
    assert len(mine) == 1 and mine[0].message.names == left and "layers.1.self_attn.rotary_emb.inv_freq" in str(mine[0].message)
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        assert check_names(model.named_params(), ck) == []          # nothing left over: no warning


def test_resident_dtypes():
    bf, f32 = torch.bfloat16, torch.float32
    assert resident_dtype(bf, bf) == bf and resident_dtype(torch.float16, bf) == bf
    assert resident_dtype(f32, bf) == f32                      # a tensor stored in 32 bits stays so
    assert resident_dtype(bf, f32) == f32 and resident_dtype(f32, f32) == f32
    assert resident_dtype(torch.int64, bf) == torch.int32 and resident_dtype(torch.uint8, f32) == torch.int32


def test_random_weights_are_a_function_of_seed_and_name(tmp_path):
    spec = ParamSpec((37, 11))
    a = random_tensor(3, "x.weight", spec, torch.float32, "cpu")
    assert torch.equal(a, random_tensor(3, "x.weight", spec, torch.float32, "cpu", chunk=50))      # piecewise = whole
    assert not torch.equal(a, random_tensor(4, "x.weight", spec, torch.float32, "cpu"))
    assert not torch.equal(a, random_tensor(3, "y.weight", spec, torch.float32, "cpu"))
    assert torch.equal(random_tensor(3, "x.weight", spec, torch.bfloat16, "cpu"), a.bfloat16())   # same values, rounded
    big = random_tensor(0, "big", ParamSpec((400, 500)), torch.float32, "cpu")
    assert abs(float(big.mean())) < 3e-4 and abs(float(big.std()) - 0.02) < 3e-4
    assert torch.equal(random_tensor(0, "n", ParamSpec((5,), init="ones"), torch.float32, "cpu"), torch.ones(5))
    f1, f2 = str(tmp_path / "a"), str(tmp_path / "b")
    write_random_model(dict(TINY_B), f1, 1, "bfloat16")
    write_random_model(dict(TINY_B), f2, 1, "bfloat16")
    c1, c2 = Checkpoint(f1), Checkpoint(f2)
    assert c1.names() == c2.names() and all(torch.equal(c1.tensor(n), c2.tensor(n)) for n in c1.names())
    assert c1.info("model.layers.1.mlp.gate.weight")[0] == torch.bfloat16
    assert torch.equal(c1.tensor("model.layers.0.input_layernorm.weight"), torch.ones(96).bfloat16())
    assert json.load(open(f1 + "/config.json"))["num_experts"] == 6
    src = RandomSource(1, torch.bfloat16, "cpu")
    src.expect(Model(build_spec(Qwen2MoeConfig.from_dict(TINY_B))).named_params())
    assert torch.equal(src.tensor("model.layers.1.mlp.gate.weight"), c1.tensor("model.layers.1.mlp.gate.weight"))
