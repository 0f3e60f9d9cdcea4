"""Fused forms of operator sequences that the reference runs as separate launches. Every function returns the
same bits as the sequence it names; none has a counterpart of its own in the reference.

    hadamard_quantize      = quantize(hadamard_transform(x))              (q8_kernels/functional/linear.py:30-31)
    rms_norm_quantize      = quantize(rms_norm_8bit(x, w)[0])             (q8_kernels/modules/attention.py:67-77)
    norm_modulate_quantize = quantize(hadamard_transform(multiply_add(rms_norm_8bit(x, w), scale, shift, 1)))
                                                                          (q8_kernels/blocks/ltx_transformer_block.py:38-40)
    flash_attn_token_major = apply_rope -> split heads -> flash_attn_func -> merge heads
                                                                          (q8_kernels/modules/attention.py:84-105)
"""
import math
from typing import Optional, Tuple

import torch

from .. import _C
from . import rope as _rope

_FP8 = torch.float8_e4m3fn


def hadamard_quantize(x: torch.Tensor, out_type: Optional[torch.dtype] = None,
                      scale: Optional[float] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """bfloat16 or e4m3 x (..., dim) -> (codes, scales) of the Hadamard-rotated rows; out_type None -> int8. The
    transform's intermediate result is rounded to x's dtype, as hadamard_transform(x) stores it."""
    if scale is None:
        scale = 1.0 / math.sqrt(x.shape[-1])
    codes, scales = _C.fht_quant(x, scale, out_type, mid_type=x.dtype)
    return codes, scales


def can_fuse_hadamard_quantize(x: torch.Tensor) -> bool:
    """The fused kernel reproduces the two-kernel sequence for bfloat16 / e4m3 inputs whose rows need no padding."""
    return x.dtype in (torch.bfloat16, _FP8) and x.shape[-1] % 8 == 0 and x.shape[-1] <= 32768


def rms_norm_quantize(x: torch.Tensor, weights: Optional[torch.Tensor] = None,
                      out_type: Optional[torch.dtype] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """bfloat16 x -> (codes, scales) of rms_norm(x) * weights; out_type None -> int8."""
    codes, scales, _ = _C.rms_norm_quant(x, weights, out_type)
    return codes, scales


def norm_modulate_quantize(x: torch.Tensor, norm_weight: Optional[torch.Tensor], mod_scale: torch.Tensor,
                           mod_shift: torch.Tensor, scale_add: float = 1.0,
                           out_type: Optional[torch.dtype] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """quantize(hadamard_transform(multiply_add(rms_norm_8bit(x, norm_weight), mod_scale, mod_shift, scale_add))) in one
    kernel: the input of an int8 projection behind an AdaLN-modulated norm
    (q8_kernels/blocks/ltx_transformer_block.py:38-40 + q8_kernels/functional/linear.py:30-31), same bits.
    x [B, T, dim] bfloat16; mod_scale / mod_shift [B, 1 or T, dim] bfloat16."""
    codes, scales = _C.norm_mod_fht_quant(x, True, norm_weight, mod_scale, mod_shift, scale_add,
                                          1.0 / math.sqrt(x.shape[-1]), out_type)
    return codes, scales


def qk_hadamard_scale(head_dim: int, softmax_scale: Optional[float] = None) -> float:
    """The factor flash_attn_func folds into the Hadamard transform of q and k when apply_qk_hadamard is set
    (q8_kernels/functional/flash_attention.py:47-51): sqrt(1 / D) * sqrt(softmax_scale)."""
    if softmax_scale is None:
        softmax_scale = head_dim ** (-0.5)
    return math.sqrt(1 / head_dim) * math.sqrt(softmax_scale)


def flash_attn_token_major(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, num_heads: int,
                           softmax_scale: Optional[float] = None, batch_mask: Optional[torch.Tensor] = None,
                           apply_qk_hadamard: bool = False, freqs_cis=None, out_dtype: Optional[torch.dtype] = None,
                           per_token_scales: bool = False, q_norm_weight: Optional[torch.Tensor] = None,
                           k_norm_weight: Optional[torch.Tensor] = None, v_codes: Optional[torch.Tensor] = None,
                           p_unit_range: bool = False, q_codes: Optional[torch.Tensor] = None) -> torch.Tensor:
    """q [B, M, H*64], k, v [B, N, H*64] bfloat16 projections (strided slices of a fused projection are read in
    place) -> attention output [B, M, H*64].

    v_codes (instead of v, which is then None; direct casts only): the e4m3 V operand [B, H, N, 64] that the QKV
    projection's GEMM wrote itself (_C.mm_bias_qkv); the prologue then handles q and k only.

    q_codes (instead of q, which is then None; direct casts with apply_qk_hadamard, no rotation, no q-norm): the e4m3 Q
    operand [B, H, M, 64] that the query projection's GEMM wrote itself (_C.mm_bias_qkv with v_col0 = 0 and
    fht_scale = qk_hadamard_scale(64, softmax_scale)); k and v [B, N, H*64] then go through one prologue launch.

    q_norm_weight / k_norm_weight (fp32 [H*64]) apply the qk-RMSNorm (over all heads of a token, no epsilon) first;
    freqs_cis = (cos, sin) fp32 tables of q's shape then rotates q and k (k must then have q's shape); they go
    through rope.compact_freqs_cis, or may be given in one of its compact forms.
    Without per_token_scales the operands are cast to e4m3 exactly as flash_attn_func does; with it each
    (token, head) row of q, k and v gets its own absmax scale. p_unit_range as in flash_attn_func (the reference's
    probability grid)."""
    d = (q_codes if q is None else q).shape[-1] // (1 if q is None else num_heads)
    if softmax_scale is None:
        softmax_scale = d ** (-0.5)
    # the tables with their repeated values stored once (same bits, a quarter of the bytes when both properties hold)
    cos, sin = (None, None) if freqs_cis is None else _rope.compact_freqs_cis(*freqs_cis)
    if apply_qk_hadamard:
        qk_scale, kernel_scale = math.sqrt(1 / d) * math.sqrt(softmax_scale), 1.0
    else:
        qk_scale, kernel_scale = 1.0, softmax_scale
    if q_codes is not None:
        if (q is not None or per_token_scales or not apply_qk_hadamard or freqs_cis is not None or q_norm_weight is not None
                or v_codes is not None or d != 64 or k.shape != v.shape or q_codes.dtype != _FP8):
            raise RuntimeError("flash_attn_token_major: q_codes replaces q for direct casts with apply_qk_hadamard, head dim 64, "
                               "no rotation and no q-norm")
        kc, vc = _C.attn_prep_kv(k, v, num_heads, None, None, True, qk_scale, False, norm_weight=k_norm_weight)
        return _C.flash_attention(q_codes, kc, vc, kernel_scale, batch_mask, out_dtype=out_dtype, token_major_out=True,
                                  p_unit_range=p_unit_range, v_token_major=True)
    if v_codes is not None:
        if per_token_scales or v is not None or d != 64 or q.shape != k.shape:
            raise RuntimeError("flash_attn_token_major: v_codes replaces v for direct casts of a self-attention with head dim 64")
        qc, kc = _C.attn_prep_qk_pair(q, k, num_heads, cos, sin, apply_qk_hadamard, qk_scale, False,
                                      q_norm_weight=q_norm_weight, k_norm_weight=k_norm_weight)
        return _C.flash_attention(qc, kc, v_codes, kernel_scale, batch_mask, out_dtype=out_dtype, token_major_out=True, p_unit_range=p_unit_range,
                                  v_token_major=True)
    if q.shape == k.shape == v.shape and d == 64:
        # self-attention: one pass over the three projections (the tables are read once, V is only cast and stays
        # token-major; the attention kernels turn its tiles while reading them from LDS).
        qc, kc, vc = _C.attn_prep_qkv(q, k, v, num_heads, cos, sin, apply_qk_hadamard, qk_scale, per_token_scales,
                                      q_norm_weight=q_norm_weight, k_norm_weight=k_norm_weight)
        if per_token_scales:
            (qc, qs), (kc, ks), (vc, vs) = qc, kc, vc
            return _C.flash_attention(qc, kc, vc, kernel_scale, batch_mask, out_dtype=out_dtype, q_scales=qs, k_scales=ks,
                                      v_scales=vs, token_major_out=True, p_unit_range=p_unit_range, v_token_major=True)
        return _C.flash_attention(qc, kc, vc, kernel_scale, batch_mask, out_dtype=out_dtype, token_major_out=True, p_unit_range=p_unit_range,
                                  v_token_major=True)
    if k.shape == v.shape and d == 64:
        # other queries than keys (cross-attention): the queries alone, keys and values together in a second launch, V
        # token-major again
        qc = _C.attn_prep_qk(q, num_heads, cos, sin, apply_qk_hadamard, qk_scale, per_token_scales,
                             norm_weight=q_norm_weight)
        kc, vc = _C.attn_prep_kv(k, v, num_heads, cos, sin, apply_qk_hadamard, qk_scale, per_token_scales,
                                 norm_weight=k_norm_weight)
        if per_token_scales:
            (qc, qs), (kc, ks), (vc, vs) = qc, kc, vc
            return _C.flash_attention(qc, kc, vc, kernel_scale, batch_mask, out_dtype=out_dtype, q_scales=qs, k_scales=ks,
                                      v_scales=vs, token_major_out=True, p_unit_range=p_unit_range, v_token_major=True)
        return _C.flash_attention(qc, kc, vc, kernel_scale, batch_mask, out_dtype=out_dtype, token_major_out=True, p_unit_range=p_unit_range,
                                  v_token_major=True)
    if q.shape == k.shape:  # one pass over q and k
        qc, kc = _C.attn_prep_qk_pair(q, k, num_heads, cos, sin, apply_qk_hadamard, qk_scale, per_token_scales,
                                      q_norm_weight=q_norm_weight, k_norm_weight=k_norm_weight)
    else:
        qc = _C.attn_prep_qk(q, num_heads, cos, sin, apply_qk_hadamard, qk_scale, per_token_scales,
                             norm_weight=q_norm_weight)
        kc = _C.attn_prep_qk(k, num_heads, cos, sin, apply_qk_hadamard, qk_scale, per_token_scales,
                             norm_weight=k_norm_weight)
    vc = _C.attn_prep_v(v, num_heads, per_token_scales)
    if per_token_scales:
        (qc, qs), (kc, ks), (vc, vs) = qc, kc, vc
        return _C.flash_attention(qc, kc, vc, kernel_scale, batch_mask, out_dtype=out_dtype, q_scales=qs, k_scales=ks,
                                  v_scales=vs, token_major_out=True, p_unit_range=p_unit_range)
    return _C.flash_attention(qc, kc, vc, kernel_scale, batch_mask, out_dtype=out_dtype, token_major_out=True, p_unit_range=p_unit_range)
