from .activations import GELU  # noqa: F401
from .attention import Attention  # noqa: F401
from .ffn import FeedForward  # noqa: F401
from .linear import FP8Linear, Q8Linear, Q8LinearLora  # noqa: F401
from .rms_norm import RMSNorm  # noqa: F401
