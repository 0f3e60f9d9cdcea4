"""Fast Walsh-Hadamard transform (reference: q8_kernels/functional/fast_hadamard.py:11-38)."""
import math
from typing import Optional

import torch

from .._C import fast_hadamard_transform


class HadamardTransformFn(torch.autograd.Function):
    """y = x H_N * scale. H_N is symmetric, so the gradient is the same transform of the incoming gradient with the
    same scale (q8_kernels/functional/fast_hadamard.py:11-22); it is returned in x's dtype and shape."""

    @staticmethod
    def forward(ctx, x, scale=1.0, out_type=None):
        ctx.scale, ctx.x_dtype = scale, x.dtype
        return fast_hadamard_transform(x, scale, out_type)

    @staticmethod
    def backward(ctx, dout):
        g = dout if dout.dtype in (torch.bfloat16, torch.float8_e4m3fn) else dout.to(torch.bfloat16)
        out_type = ctx.x_dtype if ctx.x_dtype in (torch.bfloat16, torch.float8_e4m3fn) else torch.bfloat16
        return fast_hadamard_transform(g.contiguous(), ctx.scale, out_type).to(ctx.x_dtype), None, None


def hadamard_transform(x: torch.Tensor, scale: Optional[float] = None,
                       out_type: Optional[torch.dtype] = None) -> torch.Tensor:
    """x (..., dim) -> x @ H_N * scale on the last dim, H_N the Sylvester Hadamard matrix of the next
    power of two N >= dim (x is implicitly zero-padded). scale defaults to 1/sqrt(dim) with the
    unpadded dim; out_type defaults to x.dtype. Differentiable in x."""
    if scale is None:
        scale = 1.0 / math.sqrt(x.shape[-1])
    if torch.is_grad_enabled() and x.requires_grad:
        return HadamardTransformFn.apply(x, scale, out_type)
    return fast_hadamard_transform(x, scale, out_type)
