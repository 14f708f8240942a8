"""MI355X-native quantized fused-MoE path behind vLLM-Kunlun's plugin and operator surface.

Importing the package loads libkmoe.so (hand-written gfx950 HIP kernels behind a
C ABI) and registers the torch.ops._C.moe_* operators with the reference's
names and argument order. There is no CPU or torch fallback: a missing library
is an ImportError.
"""
from . import _lib  # noqa: F401  (loads libkmoe.so or raises)
from .ops import _custom_ops  # noqa: F401  (registers torch.ops._C.*)

__version__ = "0.1.0"
