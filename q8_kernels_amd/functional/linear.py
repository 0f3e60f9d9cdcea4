"""int8 / fp8 linear layers on the 8-bit GEMM (reference: q8_kernels/functional/linear.py:22-196).

Operands that arrive in 16-bit (or fp8 for the int8 path) are quantized on the fly: int8 path = FHT rotation
then per-row int8; fp8 path = optional FHT then per-row e4m3. The backward functions return the gradient of
the activation only (the 8-bit weights are frozen), computed like the reference's with an fp8 GEMM on the
re-quantized, dequantized weight; the LoRA variant also returns the gradients of the two adapter matrices.
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


def _rotate_quant(t, out_type=None):
    """quantize(hadamard_transform(t)); one kernel where that gives the bits of the two."""
    if can_fuse_hadamard_quantize(t):
        return hadamard_quantize(t, out_type)
    return (quantize if out_type is None else quantize_fp8)(hadamard_transform(t))


def _needs_grad(t) -> bool:
    return torch.is_grad_enabled() and isinstance(t, torch.Tensor) and t.requires_grad


class GeluFn(torch.autograd.Function):
    """tanh-GELU on the gelu_forward / gelu_backward kernels (csrc/ops/gelu_forward_cuda.cu, gelu_backward_cuda.cu of the
    reference): what a fused-GELU linear falls back to when its input needs a gradient."""

    @staticmethod
    def forward(ctx, x, out_dtype):
        ctx.save_for_backward(x)
        ctx.out_dtype = out_dtype
        return _C.gelu_forward(x.contiguous(), out_dtype)

    @staticmethod
    def backward(ctx, grad_output):
        (x,) = ctx.saved_tensors
        return _C.gelu_backward(x.contiguous(), grad_output.to(x.dtype).contiguous(), ctx.out_dtype).to(x.dtype), None


# ----------------------------------------------------------------------------- int8

def _gated_residual(out, residual, gate):
    """the differentiable form of the fused epilogues: out (* gate) + residual with torch operators"""
    if residual is None:
        return out
    if gate is None:
        return out + residual.reshape(out.shape)
    groups = gate.numel() // gate.shape[-1]
    return (out.reshape(groups, -1, out.shape[-1]) * gate.reshape(groups, 1, -1)).reshape(out.shape) + residual.reshape(out.shape)


def _q8_forward(a, b, bias, scale_a, scale_b, fuse_gelu, out_dtype, residual=None, gate=None):
    a_needs_q = a.dtype == _FP8 or is_16bit(a)
    b_needs_q = b.dtype == _FP8 or is_16bit(b)
    assert (a_needs_q and scale_a is None) or (a.dtype == torch.int8 and scale_a is not None), \
        "Q8LinearFunc: a dtype missmatch"
    assert (b_needs_q and scale_b is None) or (b.dtype == torch.int8 and scale_b is not None), \
        "Q8LinearFunc: b dtype missmatch"
    assert a.shape[-1] == b.shape[-1], "Q8LinearFunc: mnk missmatch"
    assert bias is None or bias.dtype == torch.float, "Q8LinearFunc: bias must be in fp32"
    if a_needs_q:
        a, scale_a = _rotate_quant(a)
    if b_needs_q:
        b, scale_b = _rotate_quant(b)
    if bias is not None:
        out = _C.q8_mm_bias(a, b, bias, scale_a, scale_b, fuse_gelu, out_dtype, residual=residual, gate=gate)
    else:
        out = _C.q8_mm(a, b, scale_a, scale_b, fuse_gelu, out_dtype, residual=residual, gate=gate)
    return out, b, scale_b


def _grad_through_weight(grad_output, w, out_dtype):
    """grad_output [.., N] @ w [N, K] on the fp8 GEMM: both operands re-quantized per row to e4m3
    (q8_kernels/functional/linear.py:49-52)."""
    g8, gs = quantize_fp8(grad_output)
    w8, ws = quantize_fp8(w.T.contiguous())
    return _C.fp8_mm(g8, w8, gs, ws, False, out_dtype)


class Q8LinearFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, a, b, bias, scale_a, scale_b, fuse_gelu, out_dtype):
        out, bq, sb = _q8_forward(a, b, bias, scale_a, scale_b, fuse_gelu, out_dtype)
        ctx.save_for_backward(bq, sb)
        ctx.out_dtype = out_dtype
        ctx.a_shape = a.shape
        return out

    @staticmethod
    def backward(ctx, grad_output):
        # y = (a H) W'^T with W' the rotated, dequantized weight, so da = (dy W') H (H is symmetric)
        b, scale_b = ctx.saved_tensors
        w = b.to(ctx.out_dtype) * scale_b[:, None].to(ctx.out_dtype)
        grad_x = hadamard_transform(_grad_through_weight(grad_output, w, ctx.out_dtype))
        return grad_x.reshape(ctx.a_shape), None, None, None, None, None, None


def q8_linear(a: torch.Tensor, b: torch.Tensor, bias: Optional[torch.Tensor] = None,
              scale_a: Optional[torch.Tensor] = None, scale_b: Optional[torch.Tensor] = None,
              fuse_gelu: bool = False, out_dtype: Optional[torch.dtype] = None,
              residual: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """a [..., K] x b [N, K] -> [batch, M, N] through the int8 GEMM; out_dtype None -> e4m3 (as the reference).
    `residual` (bfloat16, the output's shape, out_dtype bfloat16) returns `residual + linear(a)` with the addition done
    in the GEMM's epilogue: the bits of the separate bfloat16 addition. With `gate` (bfloat16 [B, 1, N]) it returns
    `linear(a) * gate + residual`, one fused multiply-add on the bfloat16 projection (the gated residual of an AdaLN block)."""
    if _needs_grad(a):
        if fuse_gelu and out_dtype is not None and is_16bit(out_dtype):
            # the reference's backward ignores a fused GELU (functional/linear.py:44-52); here the activation follows as
            # its own differentiable step
            out = GeluFn.apply(Q8LinearFunc.apply(a, b, bias, scale_a, scale_b, False, out_dtype), out_dtype)
        else:
            out = Q8LinearFunc.apply(a, b, bias, scale_a, scale_b, fuse_gelu, out_dtype)
        return _gated_residual(out, residual, gate)
    return _q8_forward(a, b, bias, scale_a, scale_b, fuse_gelu, out_dtype, residual, gate)[0]


# ----------------------------------------------------------------------------- fp8

def _fp8_forward(a, b, bias, scale_a, scale_b, use_hadamard, out_dtype, fuse_gelu, residual=None, gate=None):
    assert (is_16bit(a) and scale_a is None) or (a.dtype == _FP8 and scale_a is not None), \
        "FP8LinearFunc: a dtype missmatch"
    assert (is_16bit(b) and scale_b is None) or (b.dtype == _FP8 and scale_b is not None), \
        "FP8LinearFunc: b dtype missmatch"
    assert a.shape[-1] == b.shape[-1], "FP8LinearFunc: mnk missmatch"
    assert bias is None or bias.dtype == torch.float, "FP8LinearFunc: bias must be in fp32"
    assert out_dtype is not None and is_16bit(out_dtype), "FP8LinearFunc: out_dtype must be in 16bit"

    def quant(t):
        return _rotate_quant(t, _FP8) if use_hadamard else quantize_fp8(t)

    if is_16bit(a):
        a, scale_a = quant(a)
    if is_16bit(b):
        b, scale_b = quant(b)
    if bias is not None:
        out = _C.fp8_mm_bias(a, b, bias, scale_a, scale_b, fuse_gelu, out_dtype, residual=residual, gate=gate)
    else:
        out = _C.fp8_mm(a, b, scale_a, scale_b, fuse_gelu, out_dtype, residual=residual, gate=gate)
    return out, b, scale_b


class FP8LinearFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, a, b, bias, scale_a, scale_b, out_dtype, use_hadamard):
        out, bq, sb = _fp8_forward(a, b, bias, scale_a, scale_b, use_hadamard, out_dtype, False)
        ctx.save_for_backward(bq, sb)
        ctx.out_dtype = out_dtype
        ctx.use_hadamard = use_hadamard
        ctx.a_shape = a.shape
        return out

    @staticmethod
    def backward(ctx, grad_output):
        b, scale_b = ctx.saved_tensors
        w = b.to(ctx.out_dtype) * scale_b[:, None].to(ctx.out_dtype)
        grad_x = _grad_through_weight(grad_output, w, ctx.out_dtype)
        if ctx.use_hadamard:  # the forward rotated a: rotate the gradient back
            grad_x = hadamard_transform(grad_x)
        return grad_x.reshape(ctx.a_shape), None, None, None, None, None, None


def fp8_linear(a: torch.Tensor, b: torch.Tensor, bias: Optional[torch.Tensor] = None,
               scale_a: Optional[torch.Tensor] = None, scale_b: Optional[torch.Tensor] = None,
               use_hadamard: bool = False, out_dtype: Optional[torch.dtype] = None, *,
               fuse_gelu: bool = False, residual: Optional[torch.Tensor] = None,
               gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """a [..., K] x b [N, K] -> [batch, M, N] through the fp8 GEMM; out_dtype must be 16-bit.

    Keyword-only extensions (defaults = the reference's behaviour): `fuse_gelu` applies tanh-GELU in the epilogue;
    `residual` (bfloat16, the output's shape) returns `residual + linear(a)` with the addition done in the epilogue;
    with `gate` (bfloat16 [B, 1, N]) `linear(a) * gate + residual` as one fused multiply-add."""
    if _needs_grad(a):  # the fused epilogues carry no gradient: GELU and the residual addition follow as separate steps
        out = FP8LinearFunc.apply(a, b, bias, scale_a, scale_b, out_dtype, use_hadamard)
        if fuse_gelu:
            out = GeluFn.apply(out, out_dtype)
        return _gated_residual(out, residual, gate)
    return _fp8_forward(a, b, bias, scale_a, scale_b, use_hadamard, out_dtype, fuse_gelu, residual, gate)[0]


# ----------------------------------------------------------------------------- int8 base weight + 16-bit LoRA

class Q8LinearLora(torch.autograd.Function):
    """o = q8_mm(quant(H a), W') (+ bias) + (a lora_a^T) lora_b^T, optionally followed by tanh-GELU
    (q8_kernels/functional/linear.py:56-133). a must be 16-bit here (the adapter branch reads it)."""

    @staticmethod
    def forward(ctx, a, b, bias, scale_a, scale_b, lora_a, lora_b, fuse_gelu, use_hadamard, out_dtype):
        assert is_16bit(a) and scale_a is None, "Q8LinearFuncLora: a must be 16bit"
        assert ((b.dtype == _FP8 or is_16bit(b)) and scale_b is None) or (b.dtype == torch.int8 and scale_b is not None), \
            "Q8LinearFuncLora: b dtype missmatch"
        assert a.shape[-1] == b.shape[-1], "Q8LinearFuncLora: mnk missmatch"
        assert bias is None or bias.dtype == torch.float, "Q8LinearFuncLora: bias must be in fp32"
        assert lora_a is not None and lora_b is not None, "Q8LinearFuncLora: lora_a and lora_b must be provided"
        assert is_16bit(lora_a) and is_16bit(lora_b), "Q8LinearFuncLora: lora_a and lora_b must be in 16bit"
        assert lora_a.shape[0] == lora_b.shape[-1], "Q8LinearFuncLora: lora_a and lora_b shape missmatch"
        assert out_dtype is not None and is_16bit(out_dtype), "Q8LinearFuncLora: out_dtype must be float16 or bfloat16"
        # the forward always rotates both operands (q8_kernels/functional/linear.py:74-77): an int8 weight is taken to
        # hold the rotated matrix, as Q8Linear.from_linear and convert_state_dict store it; use_hadamard only says
        # whether the backward rotates the gradient back (:115-128)
        a_q, sa = _rotate_quant(a)
        if b.dtype != torch.int8:
            b, scale_b = _rotate_quant(b)
        if bias is not None:
            base = _C.q8_mm_bias(a_q, b, bias, sa, scale_b, False, out_dtype)
        else:
            base = _C.q8_mm(a_q, b, sa, scale_b, False, out_dtype)
        lora_y = torch.nn.functional.linear(torch.nn.functional.linear(a, lora_a), lora_b)
        o = base + lora_y.reshape(base.shape).to(out_dtype)
        ctx.fuse_gelu, ctx.out_dtype, ctx.use_hadamard = fuse_gelu, out_dtype, use_hadamard
        ctx.a_shape = a.shape
        if fuse_gelu:
            ctx.save_for_backward(o, a, b, scale_b, lora_a, lora_b)
            return _C.gelu_forward(o, out_dtype)
        ctx.save_for_backward(None, a, b, scale_b, lora_a, lora_b)
        return o

    @staticmethod
    def backward(ctx, grad_output):
        o, a, b, scale_b, lora_a, lora_b = ctx.saved_tensors
        out_dtype = ctx.out_dtype
        if ctx.fuse_gelu:
            grad_output = _C.gelu_backward(o, grad_output.to(out_dtype).contiguous(), out_dtype)
        grad_output = grad_output.reshape(a.shape[:-1] + (grad_output.shape[-1],))
        g_lb = grad_output @ lora_b  # [.., d] @ [d, r]
        w = b.to(out_dtype) * scale_b[:, None].to(out_dtype)
        grad_x = _grad_through_weight(grad_output, w, out_dtype).reshape(ctx.a_shape)
        if ctx.use_hadamard:
            grad_x = hadamard_transform(grad_x)
        grad_x = grad_x + g_lb @ lora_a
        a2 = a.reshape(-1, a.shape[-1])
        g2 = grad_output.reshape(-1, grad_output.shape[-1])
        glb2 = g_lb.reshape(-1, g_lb.shape[-1])
        grad_lora_a = glb2.T @ a2                  # [r, h]
        grad_lora_b = g2.T @ (a2 @ lora_a.T)       # [d, r]
        return grad_x, None, None, None, None, grad_lora_a, grad_lora_b, None, None, None


def q8_linear_lora(a: torch.Tensor, b: torch.Tensor, bias: Optional[torch.Tensor] = None,
                   scale_a: Optional[torch.Tensor] = None, scale_b: Optional[torch.Tensor] = None,
                   lora_a: Optional[torch.Tensor] = None, lora_b: Optional[torch.Tensor] = None,
                   fuse_gelu: bool = False, use_hadamard: bool = True,
                   out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    return Q8LinearLora.apply(a, b, bias, scale_a, scale_b, lora_a, lora_b, fuse_gelu, use_hadamard, out_dtype)
