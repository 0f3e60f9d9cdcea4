"""Fast Walsh-Hadamard transform (reference: q8_kernels/functional/fast_hadamard.py:24-38)."""
import math
from typing import Optional

import torch

from .._C import fast_hadamard_transform


def hadamard_transform(x: torch.Tensor, scale: Optional[float] = None,
                       out_type: Optional[torch.dtype] = None) -> torch.Tensor:
    """x (..., dim) -> x @ H_N * scale on the last dim, H_N the Sylvester Hadamard matrix of the next
    power of two N >= dim (x is implicitly zero-padded). scale defaults to 1/sqrt(dim) with the
    unpadded dim; out_type defaults to x.dtype."""
    if scale is None:
        scale = 1.0 / math.sqrt(x.shape[-1])
    return fast_hadamard_transform(x, scale, out_type)
