from . import fast_hadamard, flash_attention, fma, fused, linear, quantizer, rms_norm, rope  # noqa: F401
