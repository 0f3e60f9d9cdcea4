"""Feed-forward block: fused-GELU up projection then down projection
(reference: q8_kernels/modules/ffn.py:10-17)."""
import torch.nn as nn

from .activations import GELU
from .linear import Q8Linear


class FeedForward(nn.Module):
    def __init__(self, dim: int, mult: int = 4, bias: bool = True):
        super().__init__()
        self.inner_dim = dim * mult
        self.act = GELU(dim, self.inner_dim, bias=bias)
        self.proj_down = Q8Linear(self.inner_dim, dim, bias=bias)

    def forward(self, x, out_dtype=None, x_scales=None, residual=None, gate=None):
        """residual / gate (extensions, see Q8Linear.forward): returns ff(x) (* gate) + residual from the down projection's epilogue"""
        return self.proj_down(self.act(x, out_dtype=out_dtype, x_scales=x_scales), out_dtype=out_dtype, residual=residual,
                              gate=gate)
