"""GELU projection: a Q8Linear whose GEMM epilogue applies tanh-GELU
(reference: q8_kernels/modules/activations.py:9-16)."""
import torch.nn as nn

from .linear import Q8Linear


class GELU(nn.Module):
    def __init__(self, dim_in: int, dim_out: int, approximate: str = "none", bias: bool = True):
        super().__init__()
        self.proj = Q8Linear(dim_in, dim_out, bias=bias)

    def forward(self, hidden_states, out_dtype=None, x_scales=None):
        """x_scales: row scales of an already rotated and int8-quantized hidden_states (passed on to Q8Linear)."""
        return self.proj(hidden_states, x_scales, fuse_gelu=True, out_dtype=out_dtype)
