"""FP8 flash attention forward with optional Hadamard rotation of Q and K
(reference: q8_kernels/functional/flash_attention.py:18-73)."""
import math
from typing import Optional

import torch
import torch.nn.functional as F

from .. import _C
from .fast_hadamard import hadamard_transform

_FP8 = torch.float8_e4m3fn


def _is_16bit(x) -> bool:
    return x.dtype in (torch.float16, torch.bfloat16)


def _pad_last(t: torch.Tensor, pad: int) -> torch.Tensor:
    if t.dtype == _FP8:  # zero bytes are +0.0 in e4m3
        return F.pad(t.view(torch.uint8), [0, pad]).view(_FP8)
    return F.pad(t, [0, pad])


def flash_attn_func(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, softmax_scale: Optional[float] = None,
                    batch_mask: Optional[torch.Tensor] = None, apply_qk_hadamard: bool = False, *,
                    out_dtype: Optional[torch.dtype] = None, p_unit_range: bool = False) -> torch.Tensor:
    """q [B,H,M,D], k, v [B,H,N,D] (or v already transposed to [B,H,D,N]); 16-bit inputs are cast to e4m3
    (Q and K through the FHT when apply_qk_hadamard, with the softmax scale folded into both).
    batch_mask: int32 [B] valid KV lengths. Returns [B,H,M,D]; e4m3 like the reference unless `out_dtype`
    (keyword only) asks for bfloat16. `p_unit_range=True` (keyword only) rounds the probabilities exactly on the
    reference's grid, e4m3(p) with p <= 1 (csrc/flash_attention/flash_attention_cuda.cu:197-221); the default rounds
    e4m3(2^8 p), which keeps weights down to 2^-14 of the row maximum instead of flushing those below 2^-10 to zero."""
    if softmax_scale is None:
        softmax_scale = q.shape[-1] ** (-0.5)
    head_size_og = q.size(3)
    if head_size_og % 32 != 0:
        pad = 32 - head_size_og % 32
        q, k, v = _pad_last(q, pad), _pad_last(k, pad), _pad_last(v, pad)
    assert batch_mask is None or (batch_mask.shape[0] == q.shape[0] and batch_mask.ndim == 1)
    assert k.shape[2] == v.shape[2], "v tokens != k tokens"

    if v.shape == k.shape:
        v = v.transpose(2, 3).contiguous()  # b h s d -> b h d s
    if v.shape[-1] % 16 != 0:
        v = _pad_last(v, (v.shape[-1] + 15) // 16 * 16 - v.shape[-1])
    if _is_16bit(v):
        v = v.to(_FP8)

    if apply_qk_hadamard:
        s = math.sqrt(1 / q.shape[-1]) * math.sqrt(softmax_scale)
        q = hadamard_transform(q, scale=s, out_type=_FP8)
        k = hadamard_transform(k, scale=s, out_type=_FP8)
        kernel_scale = 1.0
    else:
        q = q.to(_FP8) if _is_16bit(q) else q
        k = k.to(_FP8) if _is_16bit(k) else k
        kernel_scale = softmax_scale
    o = _C.flash_attention(q.contiguous(), k.contiguous(), v.contiguous(), kernel_scale, batch_mask, out_dtype=out_dtype,
                            p_unit_range=p_unit_range)
    return o[..., :head_size_og]
