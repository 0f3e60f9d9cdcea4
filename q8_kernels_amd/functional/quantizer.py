"""Token-wise absmax quantizers (reference: q8_kernels/functional/quantizer.py:13-17)."""
from typing import Tuple

import torch

from .._C import tokenwise_quant


def quantize(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-row int8 codes and fp32 scales (scale * code ~ x)."""
    codes, scales = tokenwise_quant(x, None)
    return codes, scales


def quantize_fp8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-row e4m3 codes (absmax mapped to 448) and fp32 scales."""
    codes, scales = tokenwise_quant(x, torch.float8_e4m3fn)
    return codes, scales
