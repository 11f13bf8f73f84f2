"""The code on either side of the operator in the reference's model: the attention module, the
transformer block, the pixel DiT and its training step, restated around this package's kernels."""
from .dit import FlowMatchingStep, LlsaSelfAttention, PixelDiT, RopeTransformerBlock

__all__ = ["PixelDiT", "RopeTransformerBlock", "LlsaSelfAttention", "FlowMatchingStep"]
