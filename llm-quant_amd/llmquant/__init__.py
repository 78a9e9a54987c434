"""llm-quant's `mode="kernel"` path on MI355X.

  core        schemes, scale computation, the quant-dequant math, the model-rewiring recipe
  quantizers  fake / real / kernel Linear modules and the `mode` lookup
  hip         loading and calling the gfx950 kernels (also importable as llmquant.cuda)
  packing     the single-file format of a quantized model
  runtime     graphed decode and the quantized KV cache
"""

from llmquant.core.config import ModelArgs, QuantConfig
from llmquant.core.modifier import QuantizationModifier
from llmquant.core.oneshot import oneshot

__all__ = ["ModelArgs", "QuantConfig", "QuantizationModifier", "oneshot"]
