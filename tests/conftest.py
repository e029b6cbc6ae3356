import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


# Two tiny configurations that differ in every size and option.
TINY_A = {
    "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe", "hidden_act": "silu",
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 4,
    "num_experts": 8, "num_experts_per_tok": 2, "norm_topk_prob": False, "moe_intermediate_size": 32,
    "shared_expert_intermediate_size": 96, "intermediate_size": 128, "decoder_sparse_step": 1,
    "mlp_only_layers": [], "vocab_size": 256, "rope_theta": 10000.0, "rms_norm_eps": 1e-6,
    "max_position_embeddings": 128, "use_sliding_window": False, "sliding_window": 32768,
    "max_window_layers": 2, "tie_word_embeddings": False,
}
TINY_B = {
    "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe", "hidden_act": "silu",
    "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 3, "num_key_value_heads": 1,
    "num_experts": 6, "num_experts_per_tok": 3, "norm_topk_prob": True, "moe_intermediate_size": 48,
    "shared_expert_intermediate_size": 64, "intermediate_size": 160, "decoder_sparse_step": 2,
    "mlp_only_layers": [0], "vocab_size": 384, "rope_theta": 1000000.0, "rms_norm_eps": 1e-5,
    "max_position_embeddings": 256, "use_sliding_window": True, "sliding_window": 16,
    "max_window_layers": 1, "tie_word_embeddings": True,
}
# a third one: GQA with groups of 2, head_dim 48, widths that are no power of two
TINY_C = {
    "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe", "hidden_act": "silu",
    "num_hidden_layers": 2, "hidden_size": 120, "num_attention_heads": 6, "num_key_value_heads": 3,
    "head_dim": 48, "num_experts": 5, "num_experts_per_tok": 1, "norm_topk_prob": True,
    "moe_intermediate_size": 40, "shared_expert_intermediate_size": 0, "intermediate_size": 72,
    "decoder_sparse_step": 1, "mlp_only_layers": [1], "vocab_size": 331, "rope_theta": 50000.0,
    "rms_norm_eps": 3e-6, "max_position_embeddings": 512, "use_sliding_window": True, "sliding_window": 40,
    "max_window_layers": 0, "tie_word_embeddings": False,
}
# layer sizes of the models the engine is built for (one layer, small vocabulary), so that the
# kernels take the code paths they take in production: head_dim 128, K = 2048 and more, 60 experts
WIDE_D = {
    "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe", "hidden_act": "silu",
    "num_hidden_layers": 1, "hidden_size": 2048, "num_attention_heads": 16, "num_key_value_heads": 16,
    "num_experts": 60, "num_experts_per_tok": 4, "norm_topk_prob": False, "moe_intermediate_size": 1408,
    "shared_expert_intermediate_size": 5632, "intermediate_size": 5632, "decoder_sparse_step": 1,
    "mlp_only_layers": [], "vocab_size": 1000, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
    "max_position_embeddings": 8192, "use_sliding_window": False, "sliding_window": 4096,
    "max_window_layers": 1, "tie_word_embeddings": False,
}
# few experts with many rows each, grouped-query attention with 7 query heads per kv head, a window
WIDE_E = {
    "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe", "hidden_act": "silu",
    "num_hidden_layers": 2, "hidden_size": 1792, "num_attention_heads": 14, "num_key_value_heads": 2,
    "num_experts": 4, "num_experts_per_tok": 2, "norm_topk_prob": True, "moe_intermediate_size": 640,
    "shared_expert_intermediate_size": 1280, "intermediate_size": 2368, "decoder_sparse_step": 1,
    "mlp_only_layers": [1], "vocab_size": 777, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
    "max_position_embeddings": 8192, "use_sliding_window": True, "sliding_window": 100,
    "max_window_layers": 1, "tie_word_embeddings": True,
}
# widths that are multiples of 4 only (no 16-byte rows), three experts, head_dim 16: the kernels' guarded paths
ODD_F = {
    "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe", "hidden_act": "silu",
    "num_hidden_layers": 2, "hidden_size": 68, "num_attention_heads": 2, "num_key_value_heads": 1,
    "head_dim": 16, "num_experts": 3, "num_experts_per_tok": 2, "norm_topk_prob": False,
    "moe_intermediate_size": 20, "shared_expert_intermediate_size": 36, "intermediate_size": 52,
    "decoder_sparse_step": 1, "mlp_only_layers": [], "vocab_size": 101, "rope_theta": 10000.0,
    "rms_norm_eps": 1e-5, "max_position_embeddings": 512, "use_sliding_window": False, "sliding_window": 64,
    "max_window_layers": 2, "tie_word_embeddings": False,
}
# every width odd (no vector load or store is aligned), one sparse and one dense layer
ODD_H = dict(ODD_F, hidden_size=71, moe_intermediate_size=21, shared_expert_intermediate_size=37, intermediate_size=51,
             vocab_size=97, mlp_only_layers=[1])
# the larger model's layer sizes with few experts: 7 query heads per kv head, eight experts per token, a shared
# expert eight times as wide as an expert
WIDE_G = {
    "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe", "hidden_act": "silu",
    "num_hidden_layers": 1, "hidden_size": 3584, "num_attention_heads": 28, "num_key_value_heads": 4,
    "num_experts": 10, "num_experts_per_tok": 8, "norm_topk_prob": False, "moe_intermediate_size": 2560,
    "shared_expert_intermediate_size": 20480, "intermediate_size": 18944, "decoder_sparse_step": 1,
    "mlp_only_layers": [], "vocab_size": 500, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
    "max_position_embeddings": 8192, "use_sliding_window": False, "sliding_window": 4096,
    "max_window_layers": 1, "tie_word_embeddings": False,
}
# one layer of the smaller model's sizes under its real vocabulary: the head and the sampling at 151,936 columns
# sixteen kv heads of 64 on a narrow model: enough (sequence, kv head) pairs for the decode attention of some twenty
# sequences to be more blocks than the GPU has CUs, while the plain model stays fast at a few hundred positions
MANY_K = {
    "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe", "hidden_act": "silu",
    "num_hidden_layers": 1, "hidden_size": 128, "num_attention_heads": 16, "num_key_value_heads": 16, "head_dim": 64,
    "num_experts": 12, "num_experts_per_tok": 3, "norm_topk_prob": False, "moe_intermediate_size": 48,
    "shared_expert_intermediate_size": 96, "intermediate_size": 128, "decoder_sparse_step": 1, "mlp_only_layers": [],
    "vocab_size": 300, "rope_theta": 1e6, "rms_norm_eps": 1e-6, "max_position_embeddings": 2048,
    "use_sliding_window": False, "sliding_window": 4096, "max_window_layers": 0, "tie_word_embeddings": False,
}
WIDE_DV = dict(WIDE_D, vocab_size=151936)
TINY = {"DV": (WIDE_DV, 7), "A": (TINY_A, 0), "B": (TINY_B, 1), "C": (TINY_C, 2), "D": (WIDE_D, 3), "E": (WIDE_E, 4), "F": (ODD_F, 5),
        "G": (WIDE_G, 6), "H": (ODD_H, 8), "K": (MANY_K, 9)}


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory):
    """name, dtype -> folder with config.json and model.safetensors (made once a session)."""
    made = {}

    def get(name: str, dtype: str = "float32", std: float = 0.02, qk_scale: float = 1.0, **overrides) -> str:
        """`std`: spread of the random weights (0.2 gives logits that single out tokens).  `qk_scale`: the query and
        key projections (weights and biases) are multiplied by it after they are drawn, which makes attention
        peaked, so that where a key lies and how exactly it is rotated shows in the logits.  `overrides` replace
        keys of the configuration."""
        key = (name, dtype, std, qk_scale, repr(sorted(overrides.items())))
        if key not in made:
            from ferrox_amd.engine.loading import write_random_model
            cfg, seed = TINY[name]
            folder = str(tmp_path_factory.mktemp(f"tiny{name}_{dtype}"))
            import torch
            # (whoever reads the folder reads what was written; the GPU makes the large models in seconds)
            device = "cuda:0" if torch.cuda.is_available() else "cpu"
            write_random_model(dict(cfg, **overrides), folder, seed, dtype, std=std, device=device)
            if qk_scale != 1.0:
                from safetensors.torch import load_file, save_file
                path = os.path.join(folder, "model.safetensors")
                tensors = load_file(path)
                for n in tensors:
                    if ".q_proj." in n or ".k_proj." in n:
                        tensors[n] = (tensors[n].double() * qk_scale).to(tensors[n].dtype)
                save_file(tensors, path)
            made[key] = folder
        return made[key]

    return get
