"""RMSNorm module (reference: q8_kernels/modules/rms_norm.py:8-17)."""
import torch
import torch.nn as nn

from .. import functional as Q8F


class RMSNorm(nn.Module):
    def __init__(self, dim: int, elementwise_affine: bool = True, device=None):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim, dtype=torch.float, device=device)) if elementwise_affine else None

    def forward(self, x, out_dtype=None):
        return Q8F.rms_norm.rms_norm_8bit(x, self.weight, out_dtype)
