"""Dense gated feed-forward: down( act(gate x) * (up x) ), act = silu for this architecture
(ferrox-moe/src/lib.rs:655-658; dense layers: ferrox-models/src/decoder.rs:2902-2913).  The
activation is a parameter of the part and of the product's epilogue (`ops.ACTIVATIONS`)."""
from __future__ import annotations

import torch

from .. import debug, ops
from .base import FEED_FORWARDS, FeedForward, ParamSpec
from .linear import Linear, same_dtype


@FEED_FORWARDS.register("gated_mlp")
class GatedMLP(FeedForward):
    kernel_libraries = ("gemm",)

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu"):
        if activation not in ops.ACTIVATIONS:
            raise ValueError(f"activation '{activation}' is not one of {sorted(ops.ACTIVATIONS)}")
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.activation = activation
        self.gate_up = self.down = None

    def param_specs(self):
        H, I = self.hidden_size, self.intermediate_size
        return {"gate_proj.weight": ParamSpec((I, H)), "up_proj.weight": ParamSpec((I, H)),
                "down_proj.weight": ParamSpec((H, I))}

    def load(self, fetch):
        self.gate_up = Linear(torch.cat(same_dtype([fetch("gate_proj.weight"), fetch("up_proj.weight")]), dim=0))
        self.down = Linear(fetch("down_proj.weight"))

    def output(self, x):
        """The feed-forward's output as float32 [T, H], added to nothing."""
        return self.down(self.gate_up(x, epilogue=ops.EPI_GATED, activation=self.activation), epilogue=ops.EPI_STORE_F32)

    def forward(self, x, ctx, residual, row_scale=None) -> None:
        debug.region("mlp gate/up")
        act = self.gate_up(x, epilogue=ops.EPI_GATED, activation=self.activation)
        debug.region("mlp down")
        self.down(act, epilogue=ops.EPI_RESID, out=residual, row_scale=row_scale)


@FEED_FORWARDS.register("swiglu")
class SwiGLU(GatedMLP):
    """The gated feed-forward with silu, under the name this architecture's description uses."""

    def __init__(self, hidden_size: int, intermediate_size: int):
        super().__init__(hidden_size, intermediate_size, "silu")
