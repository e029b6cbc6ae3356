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

    def __init__(self, vocab_size: int, hidden_size: int, tied_to: str | None = None):
        """`tied_to`: the full name of another part's [vocab, hidden] tensor that serves as this head's matrix (the
        embedding table of a model with tied embeddings); the head then has no tensor of its own."""
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.tied_to = tied_to or None
        self.weight = None

    def param_specs(self):
        return {} if self.tied_to else {"weight": ParamSpec((self.vocab_size, self.hidden_size))}

    def borrows(self):
        return [self.tied_to] if self.tied_to else []

    def load(self, fetch):
        self.weight = (fetch.shared(self.tied_to) if self.tied_to else fetch("weight")).contiguous()
        if tuple(self.weight.shape) != (self.vocab_size, self.hidden_size):
            raise ValueError(f"the head's matrix {self.tied_to or 'weight'} has shape {tuple(self.weight.shape)}, "
                             f"not [{self.vocab_size}, {self.hidden_size}]")

    def forward(self, x):
        """float32 logits [rows, vocab]."""
        return matmul(x, self.weight, epilogue=ops.EPI_STORE_F32)
