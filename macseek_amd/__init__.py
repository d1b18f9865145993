"""MI355X-native quantized matvec / MoE kernels over raw GGUF blocks (drop-in for MacSeek's src/kernels quant module)."""
from . import quant  # noqa: F401
