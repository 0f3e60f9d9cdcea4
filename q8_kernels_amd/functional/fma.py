"""Fused multiply-add of the AdaLN modulation (reference: q8_kernels/functional/fma.py:9-10)."""
import torch

from .._C import fma_8bit as fma


def multiply_add(x: torch.Tensor, y: torch.Tensor, z: torch.Tensor, scale_add: float = 0.0) -> torch.Tensor:
    """x * (y + scale_add) + z; x [B, T, dim] e4m3 (or bf16), y and z [B, T or 1, dim]; returns x's dtype."""
    return fma(x, y, z, scale_add)
