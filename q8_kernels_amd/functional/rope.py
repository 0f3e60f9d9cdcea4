"""Rotary embedding with full-shape fp32 tables (reference: q8_kernels/functional/rope.py:9-44).

The reference's apply_rope runs a pure-torch formula (its CUDA op is commented out); this one runs
the HIP kernels, which evaluate the same interleaved-pair formula and its transpose in fp32."""
from typing import Optional

import torch

from .._C import rope, rope_backward


class ROPE(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, cos_freqs, sin_freqs, out_type):
        ctx.save_for_backward(cos_freqs, sin_freqs)
        ctx.out_type = out_type
        return rope(x, cos_freqs, sin_freqs, out_type)

    @staticmethod
    def backward(ctx, grad_output):
        cos_freqs, sin_freqs = ctx.saved_tensors
        return rope_backward(grad_output, cos_freqs, sin_freqs, ctx.out_type), None, None, None


def apply_rope(x: torch.Tensor, cos_freqs: torch.Tensor, sin_freqs: torch.Tensor,
               out_type: Optional[torch.dtype] = None) -> torch.Tensor:
    assert x.dtype in (torch.float8_e4m3fn, torch.bfloat16), "apply_rope: x must be bf16 or e4m3"
    assert cos_freqs.dtype == torch.float and sin_freqs.dtype == torch.float, "apply_rope: tables must be fp32"
    assert cos_freqs.shape == x.shape and sin_freqs.shape == x.shape, "apply_rope: tables must match x"
    if torch.is_grad_enabled() and x.requires_grad:
        return ROPE.apply(x, cos_freqs, sin_freqs, out_type)
    return rope(x, cos_freqs, sin_freqs, out_type)
