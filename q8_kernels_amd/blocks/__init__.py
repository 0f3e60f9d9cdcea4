from .dit_block import Fp8DiTBlock  # noqa: F401
from .ltx_transformer_block import LTXTransformerBlock  # noqa: F401
