"""int8 / fp8 linear layers on the 8-bit GEMM (reference: q8_kernels/functional/linear.py:24-42,138-196).

Forward (inference) only. Operands that arrive in 16-bit (or fp8 for the int8 path) are quantized on
the fly: int8 path = FHT rotation then per-row int8; fp8 path = optional FHT then per-row e4m3.
"""
from typing import Optional

import torch

from .. import _C
from .fast_hadamard import hadamard_transform
from .fused import can_fuse_hadamard_quantize, hadamard_quantize
from .quantizer import quantize, quantize_fp8

_FP8 = torch.float8_e4m3fn


def is_16bit(x) -> bool:
    dtype = x.dtype if hasattr(x, "dtype") else x
    return dtype in (torch.float16, torch.bfloat16)


def q8_linear(a: torch.Tensor, b: torch.Tensor, bias: Optional[torch.Tensor] = None,
              scale_a: Optional[torch.Tensor] = None, scale_b: Optional[torch.Tensor] = None,
              fuse_gelu: bool = False, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """a [..., K] x b [N, K] -> [batch, M, N] through the int8 GEMM; out_dtype None -> e4m3 (as the reference)."""
    a_needs_q = a.dtype == _FP8 or is_16bit(a)
    b_needs_q = b.dtype == _FP8 or is_16bit(b)
    assert (a_needs_q and scale_a is None) or (a.dtype == torch.int8 and scale_a is not None), \
        "Q8LinearFunc: a dtype missmatch"
    assert (b_needs_q and scale_b is None) or (b.dtype == torch.int8 and scale_b is not None), \
        "Q8LinearFunc: b dtype missmatch"
    assert a.shape[-1] == b.shape[-1], "Q8LinearFunc: mnk missmatch"
    assert bias is None or bias.dtype == torch.float, "Q8LinearFunc: bias must be in fp32"
    def rotate_quant(t):  # one kernel where it gives the bits of the two
        return hadamard_quantize(t) if can_fuse_hadamard_quantize(t) else quantize(hadamard_transform(t))

    if a_needs_q:
        a, scale_a = rotate_quant(a)
    if b_needs_q:
        b, scale_b = rotate_quant(b)
    if bias is not None:
        return _C.q8_mm_bias(a, b, bias, scale_a, scale_b, fuse_gelu, out_dtype)
    return _C.q8_mm(a, b, scale_a, scale_b, fuse_gelu, out_dtype)


def fp8_linear(a: torch.Tensor, b: torch.Tensor, bias: Optional[torch.Tensor] = None,
               scale_a: Optional[torch.Tensor] = None, scale_b: Optional[torch.Tensor] = None,
               use_hadamard: bool = False, out_dtype: Optional[torch.dtype] = None, *,
               fuse_gelu: bool = False) -> torch.Tensor:
    """a [..., K] x b [N, K] -> [batch, M, N] through the fp8 GEMM; out_dtype must be 16-bit.

    `fuse_gelu` (keyword only, default False = the reference's behaviour) applies tanh-GELU in the epilogue."""
    assert (is_16bit(a) and scale_a is None) or (a.dtype == _FP8 and scale_a is not None), \
        "FP8LinearFunc: a dtype missmatch"
    assert (is_16bit(b) and scale_b is None) or (b.dtype == _FP8 and scale_b is not None), \
        "FP8LinearFunc: b dtype missmatch"
    assert a.shape[-1] == b.shape[-1], "FP8LinearFunc: mnk missmatch"
    assert bias is None or bias.dtype == torch.float, "FP8LinearFunc: bias must be in fp32"
    assert out_dtype is not None and is_16bit(out_dtype), "FP8LinearFunc: out_dtype must be in 16bit"

    def quant(t):
        if use_hadamard:
            if can_fuse_hadamard_quantize(t):
                return hadamard_quantize(t, _FP8)
            return quantize_fp8(hadamard_transform(t))
        return quantize_fp8(t)

    if is_16bit(a):
        a, scale_a = quant(a)
    if is_16bit(b):
        b, scale_b = quant(b)
    if bias is not None:
        return _C.fp8_mm_bias(a, b, bias, scale_a, scale_b, fuse_gelu, out_dtype)
    return _C.fp8_mm(a, b, scale_a, scale_b, fuse_gelu, out_dtype)
