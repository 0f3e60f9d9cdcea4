"""RMSNorm forward (reference: q8_kernels/functional/rms_norm.py:9-24)."""
from typing import Optional

import torch

from .._C import rms_norm


def rms_norm_8bit(x: torch.Tensor, weights: Optional[torch.Tensor] = None,
                  out_type: Optional[torch.dtype] = None) -> torch.Tensor:
    """x * rsqrt(mean(x^2)) * weights, no epsilon; weights must be fp32 (or None)."""
    assert weights is None or weights.dtype == torch.float, "RMSNorm8bit: dtype missmatch"
    y, _rstd = rms_norm(x, weights, out_type)
    return y
