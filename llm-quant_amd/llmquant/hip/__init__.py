"""Loading and calling the gfx950 kernels (the reference's llmquant.cuda)."""

from llmquant.hip.build import build_extension, load_capi, load_extension
from llmquant.hip.ops import fake_quantize_cuda, fake_quantize_hip, quantize_activation

__all__ = [
    "build_extension", "fake_quantize_cuda", "fake_quantize_hip", "load_capi",
    "load_extension", "quantize_activation",
]
