"""Qwen2-MoE as a list of parts.

Every layer is a pre-norm block of paged grouped-query attention (q/k/v bias,
split-half rotary over the whole head) and a feed-forward that is either the
sparse mixture (softmax router over all experts, top-k, optional
renormalisation, sigmoid-gated shared expert) or a dense gated MLP, as the
configuration's layer plan says; layers from `max_window_layers` on attend
within a sliding window.  Tensor names are those of the checkpoint
(`model.layers.N.self_attn.q_proj.weight`, ...).  The computation follows the
reference's generic decoder for this architecture
(ferrox-models/src/decoder.rs:3014-3678, capability.rs:252-258).
"""
from __future__ import annotations

from ..config.qwen2_moe import Qwen2MoeConfig
from ..parts.base import LayerSpec, ModelSpec, PartSpec, ScheduleEntry


def build_spec(cfg: Qwen2MoeConfig, tensor_names=None) -> ModelSpec:
    """`tensor_names`: names the checkpoint holds, used only where the configuration leaves a
    choice open (q/k/v bias when `qkv_bias` is not given: present iff the tensors are,
    as ferrox-models/src/loader.rs:1252-1254 decides it)."""
    H = cfg.hidden_size
    bias = cfg.qkv_bias
    if bias is None:
        bias = True if tensor_names is None else "model.layers.0.self_attn.q_proj.bias" in set(tensor_names)
    layers = []
    for l in range(cfg.num_hidden_layers):
        norm = {"size": H, "eps": cfg.rms_norm_eps}
        mixer = PartSpec("paged_attention", {
            "hidden_size": H, "n_heads": cfg.num_attention_heads, "n_kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "bias": bias, "window": cfg.layer_window(l),
            "position": PartSpec("rope_neox", {"head_dim": cfg.head_dim, "theta": cfg.rope_theta}),
        }, prefix="self_attn.")
        if cfg.layer_is_sparse(l):
            ffn = PartSpec("sparse_moe", {
                "hidden_size": H, "n_experts": cfg.num_experts, "top_k": cfg.num_experts_per_tok,
                "expert_intermediate_size": cfg.moe_intermediate_size, "norm_topk_prob": cfg.norm_topk_prob,
                "gating": "softmax", "shared_intermediate_size": cfg.shared_expert_intermediate_size,
                "shared_gate": True,
            }, prefix="mlp.")
        else:
            ffn = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": cfg.intermediate_size}, prefix="mlp.")
        layers.append(LayerSpec("prenorm", f"model.layers.{l}.", {
            "norm1": PartSpec("rmsnorm", dict(norm), prefix="input_layernorm."),
            "mixer": mixer,
            "norm2": PartSpec("rmsnorm", dict(norm), prefix="post_attention_layernorm."),
            "ffn": ffn,
        }))
    return ModelSpec(
        hidden_size=H, vocab_size=cfg.vocab_size,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab_size, "hidden_size": H},
                           prefix="model.embed_tokens."),
        layers=layers,
        schedule=[ScheduleEntry(l) for l in range(cfg.num_hidden_layers)],
        final_norm=PartSpec("rmsnorm", {"size": H, "eps": cfg.rms_norm_eps}, prefix="model.norm."),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab_size, "hidden_size": H,           # loader.rs:1433-1436
                                      "tied_to": "model.embed_tokens.weight" if cfg.tie_word_embeddings else None},
                      prefix="lm_head."),
        max_positions=cfg.max_position_embeddings,
        eos_token_id=cfg.eos_token_id,
    )
