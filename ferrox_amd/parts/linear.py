"""A weight matrix [out, in] with an optional bias, applied through the matrix
product kernels.  A weight that the checkpoint stores in float32 stays float32
even when activations are bfloat16; the product then runs in float32."""
from __future__ import annotations

import torch

from .. import ops


def matmul(x: torch.Tensor, weight: torch.Tensor, *, epilogue: int = ops.EPI_STORE, out=None, **kw) -> torch.Tensor:
    """ops.gemm, also for float32 weights under bfloat16 activations."""
    if x.dtype == weight.dtype:
        return ops.gemm(x, weight, epilogue=epilogue, out=out, **kw)
    if weight.dtype != torch.float32:
        raise ops.KernelError(f"activations {x.dtype} with weights {weight.dtype}")
    x32 = ops.cast(x, torch.float32)
    if epilogue in (ops.EPI_STORE_F32, ops.EPI_RESID):
        return ops.gemm(x32, weight, epilogue=epilogue, out=out, **kw)
    y = ops.cast(ops.gemm(x32, weight, epilogue=epilogue, **kw), x.dtype)
    if out is not None:
        out.copy_(y)
        return out
    return y


def same_dtype(tensors):
    """Tensors that are joined into one matrix must agree; float32 wins."""
    if any(t.dtype == torch.float32 for t in tensors):
        return [t.float() for t in tensors]
    return list(tensors)


class Linear:
    def __init__(self, weight: torch.Tensor, bias: torch.Tensor | None = None):
        self.weight = weight.contiguous()
        self.bias = bias

    def __call__(self, x: torch.Tensor, **kw) -> torch.Tensor:
        return matmul(x, self.weight, bias=self.bias, **kw)
