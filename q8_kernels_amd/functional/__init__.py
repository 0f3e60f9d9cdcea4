from . import fast_hadamard, flash_attention, fused, linear, quantizer, rms_norm, rope  # noqa: F401
