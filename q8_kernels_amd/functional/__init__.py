from . import fast_hadamard, flash_attention, linear, quantizer, rms_norm, rope  # noqa: F401
