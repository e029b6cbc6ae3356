"""Typed configuration of the Qwen2-MoE architecture, read from config.json.

Field meanings follow the reference's `ModelConfig` / `MoeLayerConfig`
(ferrox-models/src/config.rs:151-230, ferrox-moe/src/lib.rs:28-69); the key names
are those of the model's own config.json.  Three things the reference does not
have are read here: `norm_topk_prob` (the reference fixes it by architecture
name, ferrox-models/src/loader.rs:92,323), the plan of dense and sparse layers
(`decoder_sparse_step`, `mlp_only_layers`) and the layers a sliding window
applies to (`use_sliding_window`, `sliding_window`, `max_window_layers`).
"""
from __future__ import annotations

from dataclasses import dataclass, field

from .. import limits
from .base import ConfigError, ConfigReader


@dataclass(frozen=True)
class Qwen2MoeConfig:
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    moe_intermediate_size: int
    shared_expert_intermediate_size: int
    num_experts: int
    num_experts_per_tok: int
    norm_topk_prob: bool
    decoder_sparse_step: int
    mlp_only_layers: tuple
    rope_theta: float
    rms_norm_eps: float
    max_position_embeddings: int
    use_sliding_window: bool
    sliding_window: int
    max_window_layers: int
    tie_word_embeddings: bool
    qkv_bias: bool | None      # None: decided by whether the checkpoint holds the bias tensors
    eos_token_id: int | tuple | None = None      # one id, or several (chat variants stop on either of two)
    bos_token_id: int | None = None
    defaulted_keys: tuple = field(default=(), compare=False)

    architecture = "Qwen2MoeForCausalLM"
    model_type = "qwen2_moe"

    # ---- reading -------------------------------------------------------
    @classmethod
    def from_dict(cls, raw: dict, where: str = "config.json") -> "Qwen2MoeConfig":
        r = ConfigReader(raw, where)
        hidden = r.integer("hidden_size", minimum=1)
        heads = r.integer("num_attention_heads", minimum=1)
        kv_heads = r.integer("num_key_value_heads", heads, minimum=1)
        head_dim = r.optional_integer("head_dim", minimum=1)
        if head_dim is None:
            if hidden % heads:
                raise ConfigError(f"{where}: hidden_size {hidden} is not a multiple of "
                                  f"num_attention_heads {heads} and no head_dim is given")
            head_dim = hidden // heads
        experts = r.integer("num_experts", 0, minimum=0)
        top_k = r.integer("num_experts_per_tok", 2 if experts else 0, minimum=0)  # default 2: loader.rs:248-256
        eos = raw.get("eos_token_id")
        if isinstance(eos, list):
            if any(isinstance(i, bool) or not isinstance(i, int) for i in eos):
                raise ConfigError(f"{where}: key 'eos_token_id' must be an integer or a list of integers, got {eos!r}")
            eos = tuple(eos) if len(eos) > 1 else (eos[0] if eos else None)
        elif eos is not None and (isinstance(eos, bool) or not isinstance(eos, int)):
            raise ConfigError(f"{where}: key 'eos_token_id' must be an integer or a list of integers, got {eos!r}")
        cfg = cls(
            vocab_size=r.integer("vocab_size", minimum=1),
            hidden_size=hidden,
            num_hidden_layers=r.integer("num_hidden_layers", minimum=1),
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            intermediate_size=r.integer("intermediate_size", 0, minimum=0),
            moe_intermediate_size=r.integer("moe_intermediate_size", 0, minimum=0),
            shared_expert_intermediate_size=r.integer("shared_expert_intermediate_size", 0, minimum=0),
            num_experts=experts,
            num_experts_per_tok=top_k,
            norm_topk_prob=r.boolean("norm_topk_prob", False),
            decoder_sparse_step=r.integer("decoder_sparse_step", 1, minimum=1),
            mlp_only_layers=r.int_list("mlp_only_layers", ()),
            rope_theta=r.number("rope_theta", 10000.0, positive=True),
            rms_norm_eps=r.number("rms_norm_eps", 1e-6, positive=True),
            max_position_embeddings=r.integer("max_position_embeddings", 4096, minimum=1),  # 4096: run.rs:551-559
            use_sliding_window=r.boolean("use_sliding_window", False),
            sliding_window=r.integer("sliding_window", 0, minimum=0),
            max_window_layers=r.integer("max_window_layers", 0, minimum=0),
            tie_word_embeddings=r.boolean("tie_word_embeddings", False),
            qkv_bias=raw.get("qkv_bias") if isinstance(raw.get("qkv_bias"), bool) else None,
            eos_token_id=eos,
            bos_token_id=raw.get("bos_token_id") if isinstance(raw.get("bos_token_id"), int) else None,
            defaulted_keys=tuple(r.defaulted),
        )
        cfg._refuse_unsupported(raw, where)
        cfg.validate(where)
        return cfg

    @staticmethod
    def _refuse_unsupported(raw: dict, where: str) -> None:
        """Fail closed on features this engine does not compute, as the reference
        does for its own list (ferrox-models/src/capability.rs:616-638)."""
        if raw.get("rope_scaling") not in (None, {}):
            raise ConfigError(f"{where}: rope_scaling={raw['rope_scaling']!r} is not supported")
        act = raw.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"{where}: hidden_act={act!r} is not supported (only 'silu')")
        if raw.get("quantization_config") is not None:
            raise ConfigError(f"{where}: quantized checkpoints (quantization_config) are not supported")

    def validate(self, where: str = "config") -> None:
        def bad(msg):
            raise ConfigError(f"{where}: {msg}")

        if self.num_attention_heads % self.num_key_value_heads:         # config.rs:758-767
            bad(f"num_attention_heads {self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            bad(f"head_dim {self.head_dim} must be even for rotary pairs")
        if self.num_experts and not 1 <= self.num_experts_per_tok <= self.num_experts:
            bad(f"num_experts_per_tok {self.num_experts_per_tok} must lie in 1..num_experts {self.num_experts}")
        if self.num_experts > limits.MOE_MAX_EXPERTS:
            bad(f"num_experts {self.num_experts} is more than the routing kernels take ({limits.MOE_MAX_EXPERTS})")
        if self.num_experts_per_tok > limits.MOE_MAX_TOP_K:
            bad(f"num_experts_per_tok {self.num_experts_per_tok} is more than the routing kernels take "
                f"({limits.MOE_MAX_TOP_K})")
        if self.head_dim % limits.HEAD_DIM_STEP or self.head_dim > limits.HEAD_DIM_MAX:
            bad(f"head_dim {self.head_dim}: the attention kernels take multiples of {limits.HEAD_DIM_STEP} "
                f"up to {limits.HEAD_DIM_MAX}")
        for l in self.mlp_only_layers:
            if not 0 <= l < self.num_hidden_layers:
                bad(f"mlp_only_layers names layer {l}, the model has {self.num_hidden_layers}")
        kinds = [self.layer_is_sparse(l) for l in range(self.num_hidden_layers)]
        if any(kinds) and self.moe_intermediate_size < 1:
            bad("sparse layers need moe_intermediate_size >= 1")
        if not all(kinds) and self.intermediate_size < 1:
            bad("dense layers need intermediate_size >= 1")
        if self.use_sliding_window and self.max_window_layers < self.num_hidden_layers \
                and self.sliding_window < 1:
            bad("use_sliding_window is true but sliding_window < 1")

    # ---- the per-layer plan -----------------------------------------------
    def layer_is_sparse(self, layer: int) -> bool:
        """Layer has router and experts; otherwise a dense SwiGLU of `intermediate_size`."""
        return (layer not in self.mlp_only_layers and self.num_experts > 0
                and (layer + 1) % self.decoder_sparse_step == 0)

    def layer_window(self, layer: int):
        """Window of the layer's attention in positions, or None for all keys.
        A query at position p sees key t iff p - t < window
        (ferrox-core/src/attention.rs:498-513)."""
        if self.use_sliding_window and layer >= self.max_window_layers:
            return self.sliding_window
        return None

    @property
    def has_shared_expert(self) -> bool:
        return self.shared_expert_intermediate_size > 0

    def to_dict(self) -> dict:
        """The config.json this configuration is read back from."""
        d = {
            "architectures": [self.architecture],
            "model_type": self.model_type,
            "hidden_act": "silu",
        }
        for k in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                  "num_key_value_heads", "head_dim", "intermediate_size", "moe_intermediate_size",
                  "shared_expert_intermediate_size", "num_experts", "num_experts_per_tok",
                  "norm_topk_prob", "decoder_sparse_step", "rope_theta", "rms_norm_eps",
                  "max_position_embeddings", "use_sliding_window", "sliding_window",
                  "max_window_layers", "tie_word_embeddings"):
            d[k] = getattr(self, k)
        if self.qkv_bias is not None:
            d["qkv_bias"] = self.qkv_bias
        d["mlp_only_layers"] = list(self.mlp_only_layers)
        if self.eos_token_id is not None:
            d["eos_token_id"] = list(self.eos_token_id) if isinstance(self.eos_token_id, tuple) else self.eos_token_id
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        return d
