"""RMSNorm forward and backward (reference: q8_kernels/functional/rms_norm.py:8-24)."""
from typing import Optional

import torch

from .._C import rms_norm, rms_norm_backward


class RMSNorm8bit(torch.autograd.Function):
    """y = x * rsqrt(mean(x^2)) * weights; the backward returns dx only, like the reference (weights are frozen)."""

    @staticmethod
    def forward(ctx, x, weights, out_type):
        assert weights is None or weights.dtype == torch.float, "RMSNorm8bit: dtype missmatch"
        x_normed, x_norms = rms_norm(x, weights, out_type)
        ctx.save_for_backward(x_normed, x_norms, weights)
        ctx.out_type = out_type
        return x_normed

    @staticmethod
    def backward(ctx, grad_output):
        x_normed, x_norms, weights = ctx.saved_tensors
        return rms_norm_backward(x_normed, x_norms, grad_output, weights, ctx.out_type), None, None


def rms_norm_8bit(x: torch.Tensor, weights: Optional[torch.Tensor] = None,
                  out_type: Optional[torch.dtype] = None) -> torch.Tensor:
    """x * rsqrt(mean(x^2)) * weights, no epsilon; weights must be fp32 (or None)."""
    assert weights is None or weights.dtype == torch.float, "RMSNorm8bit: dtype missmatch"
    if torch.is_grad_enabled() and x.requires_grad:
        return RMSNorm8bit.apply(x, weights, out_type)
    return rms_norm(x, weights, out_type)[0]
