"""Configuration and registry: reading config.json keys, defaults, the layer plan, refusals."""
import json

import pytest

from conftest import TINY_A, TINY_B, TINY_C
from ferrox_amd.config import ConfigError, Qwen2MoeConfig
from ferrox_amd.models import config_from_folder, known_architectures, resolve
from ferrox_amd.models.qwen2_moe import build_spec


def test_reads_every_size_from_the_keys():
    a, b = Qwen2MoeConfig.from_dict(TINY_A), Qwen2MoeConfig.from_dict(TINY_B)
    assert (a.num_hidden_layers, a.hidden_size, a.num_attention_heads, a.num_key_value_heads, a.head_dim) == (2, 64, 4, 4, 16)
    assert (b.num_hidden_layers, b.hidden_size, b.num_attention_heads, b.num_key_value_heads, b.head_dim) == (3, 96, 3, 1, 32)
    assert (a.num_experts, a.num_experts_per_tok, a.norm_topk_prob) == (8, 2, False)
    assert (b.num_experts, b.num_experts_per_tok, b.norm_topk_prob) == (6, 3, True)
    assert (a.vocab_size, a.rope_theta, a.rms_norm_eps) == (256, 1e4, 1e-6)
    assert (b.vocab_size, b.rope_theta, b.rms_norm_eps, b.tie_word_embeddings) == (384, 1e6, 1e-5, True)
    assert Qwen2MoeConfig.from_dict(TINY_C).head_dim == 48          # an explicit head_dim wins over hidden/heads


def test_layer_plan_and_windows():
    b = Qwen2MoeConfig.from_dict(TINY_B)
    assert [b.layer_is_sparse(l) for l in range(3)] == [False, True, False]        # step 2, mlp_only [0]
    assert [b.layer_window(l) for l in range(3)] == [None, 16, 16]                # from max_window_layers = 1 on
    a = Qwen2MoeConfig.from_dict(TINY_A)
    assert all(a.layer_is_sparse(l) for l in range(2)) and all(a.layer_window(l) is None for l in range(2))
    c = Qwen2MoeConfig.from_dict(TINY_C)
    assert [c.layer_is_sparse(l) for l in range(2)] == [True, False] and [c.layer_window(l) for l in range(2)] == [40, 40]


def test_defaults_are_reported():
    raw = {"architectures": ["Qwen2MoeForCausalLM"], "hidden_size": 32, "num_attention_heads": 2,
           "num_hidden_layers": 1, "vocab_size": 10, "intermediate_size": 16}
    cfg = Qwen2MoeConfig.from_dict(raw)
    assert cfg.num_key_value_heads == 2 and cfg.rope_theta == 10000.0 and cfg.rms_norm_eps == 1e-6
    assert cfg.num_experts == 0 and not cfg.layer_is_sparse(0)
    assert {"num_key_value_heads", "rope_theta", "rms_norm_eps", "norm_topk_prob"} <= set(cfg.defaulted_keys)
    assert cfg.qkv_bias is None
    assert Qwen2MoeConfig.from_dict(cfg.to_dict()) == cfg               # round trip through config.json


@pytest.mark.parametrize("patch,word", [
    ({"hidden_size": None}, "hidden_size"),
    ({"num_attention_heads": 3, "num_key_value_heads": 2}, "multiple"),
    ({"num_experts_per_tok": 9}, "num_experts_per_tok"),
    ({"vocab_size": "big"}, "vocab_size"),
    ({"rope_scaling": {"type": "yarn", "factor": 4}}, "rope_scaling"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"quantization_config": {"bits": 4}}, "quantized"),
    ({"mlp_only_layers": [7]}, "mlp_only_layers"),
    ({"head_dim": 15}, "head_dim"),
    ({"head_dim": 24}, "head_dim"),                       # even, but no multiple of 16: refused when read, not at the first step
    ({"head_dim": 272}, "head_dim"),
    ({"num_experts": 1025}, "num_experts"),
    ({"num_experts": 64, "num_experts_per_tok": 33}, "num_experts_per_tok"),
    ({"use_sliding_window": True, "sliding_window": 0, "max_window_layers": 0}, "sliding_window"),
    ({"rms_norm_eps": -1.0}, "rms_norm_eps"),
    ({"eos_token_id": "stop"}, "eos_token_id"),
    ({"eos_token_id": [3, 4.5]}, "eos_token_id"),
])
def test_bad_configs_are_refused_with_the_key_named(patch, word):
    raw = dict(TINY_A)
    raw.update(patch)
    raw = {k: v for k, v in raw.items() if v is not None}
    with pytest.raises(ConfigError) as e:
        Qwen2MoeConfig.from_dict(raw)
    assert word in str(e.value)


def test_stop_ids_are_one_or_several():
    one = Qwen2MoeConfig.from_dict(dict(TINY_A, eos_token_id=7))
    two = Qwen2MoeConfig.from_dict(dict(TINY_A, eos_token_id=[7, 9]))
    assert one.eos_token_id == 7 and two.eos_token_id == (7, 9)
    assert Qwen2MoeConfig.from_dict(dict(TINY_A, eos_token_id=[7])).eos_token_id == 7
    assert Qwen2MoeConfig.from_dict(dict(TINY_A)).eos_token_id is None
    assert two.to_dict()["eos_token_id"] == [7, 9] and Qwen2MoeConfig.from_dict(two.to_dict()) == two
    assert build_spec(two).eos_token_id == (7, 9)


def test_registry_is_closed(tmp_path):
    assert known_architectures() == ["Qwen2MoeForCausalLM"]
    assert resolve({"architectures": ["Qwen2MoeForCausalLM"]}).model_type == "qwen2_moe"
    assert resolve({"model_type": "qwen2_moe"}).name == "Qwen2MoeForCausalLM"
    with pytest.raises(ConfigError) as e:
        resolve({"architectures": ["LlamaForCausalLM"]})
    assert "LlamaForCausalLM" in str(e.value)
    with pytest.raises(ConfigError):
        resolve({})
    (tmp_path / "config.json").write_text(json.dumps(TINY_B))
    arch, cfg = config_from_folder(str(tmp_path))
    assert arch.name == "Qwen2MoeForCausalLM" and cfg.hidden_size == 96
    with pytest.raises(ConfigError):
        config_from_folder(str(tmp_path / "nowhere"))


def test_spec_is_chosen_layer_by_layer():
    spec = build_spec(Qwen2MoeConfig.from_dict(TINY_B))
    kinds = [(l.parts["mixer"].kind, l.parts["ffn"].kind, l.parts["mixer"].args["window"]) for l in spec.layers]
    assert kinds == [("paged_attention", "swiglu", None), ("paged_attention", "sparse_moe", 16),
                     ("paged_attention", "swiglu", 16)]
    assert spec.layers[1].parts["ffn"].args["top_k"] == 3 and spec.layers[0].parts["ffn"].args["intermediate_size"] == 160
    assert spec.head.args["tied_to"] == "model.embed_tokens.weight" and [e.layer for e in spec.schedule] == [0, 1, 2]
    # q/k/v bias not stated in the config: decided by what the checkpoint holds
    assert build_spec(Qwen2MoeConfig.from_dict(TINY_B), ["model.layers.0.self_attn.q_proj.weight"]) \
        .layers[0].parts["mixer"].args["bias"] is False
