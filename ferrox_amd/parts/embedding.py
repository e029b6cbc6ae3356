"""Token embedding (no scale, ferrox-models/src/decoder.rs:1279-1284) and the output
head, applied to the wanted rows only (decoder.rs:2994-3009); a tied head shares
the embedding table (ferrox-models/src/loader.rs:1433-1436)."""
from __future__ import annotations

from .. import ops
from .base import EMBEDDINGS, HEADS, ParamSpec, Part
from .linear import matmul


@EMBEDDINGS.register("token_embedding")
class TokenEmbedding(Part):
    kernel_libraries = ("elementwise",)

    def __init__(self, vocab_size: int, hidden_size: int):
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.weight = None

    def param_specs(self):
        return {"weight": ParamSpec((self.vocab_size, self.hidden_size))}

    def load(self, fetch):
        self.weight = fetch("weight").contiguous()

    def forward(self, token_ids):
        return ops.embed(self.weight, token_ids)


@HEADS.register("linear_head")
class LinearHead(Part):
    kernel_libraries = ("gemm",)

    def __init__(self, vocab_size: int, hidden_size: int, tied: bool = False):
        self.vocab_size, self.hidden_size, self.tied = int(vocab_size), int(hidden_size), bool(tied)
        self.weight = None

    def param_specs(self):
        return {} if self.tied else {"weight": ParamSpec((self.vocab_size, self.hidden_size))}

    def load(self, fetch):
        if not self.tied:
            self.weight = fetch("weight").contiguous()

    def tie(self, embedding: TokenEmbedding):
        self.weight = embedding.weight

    def forward(self, x):
        """float32 logits [rows, vocab]."""
        return matmul(x, self.weight, epilogue=ops.EPI_STORE_F32)
