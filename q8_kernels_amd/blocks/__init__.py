from .dit_block import Fp8DiTBlock  # noqa: F401
