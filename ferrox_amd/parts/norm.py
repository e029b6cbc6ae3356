"""RMSNorm (ferrox-core/src/matmul.rs:62-69): y = x * rsqrt(mean(x^2) + eps) * w,
statistics in float32, read from the float32 residual stream."""
from __future__ import annotations

from .. import ops
from .base import NORMS, Norm, ParamSpec


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    kernel_libraries = ("elementwise",)

    def __init__(self, size: int, eps: float):
        self.size = int(size)
        self.eps = float(eps)
        self.weight = None

    def param_specs(self):
        return {"weight": ParamSpec((self.size,), init="ones")}

    def load(self, fetch):
        self.weight = fetch("weight").contiguous()

    def rms_params(self):
        return self.weight, self.eps

    def forward(self, h, ctx, rows=None):
        return ops.rmsnorm(h, self.weight, self.eps, ctx.act_dtype, rows=rows)
