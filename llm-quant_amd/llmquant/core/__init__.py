"""Shared by every stage; nothing here imports a stage at module level."""

from llmquant.core.config import BF16, DTYPE_BITS, ModelArgs, QuantConfig
from llmquant.core.modifier import QuantizationModifier
from llmquant.core.observers import SCALE_EPS, compute_scale, group_view, pad_to_group
from llmquant.core.oneshot import oneshot
from llmquant.core.quant_ops import dequantize, fake_quantize, quantize
from llmquant.core.scheme import (
    GROUP_SIZE,
    PRESET_SCHEMES,
    QuantizationArgs,
    QuantizationScheme,
    preset_name_to_scheme,
)

__all__ = [
    "BF16", "DTYPE_BITS", "GROUP_SIZE", "PRESET_SCHEMES", "SCALE_EPS", "ModelArgs",
    "QuantConfig", "QuantizationArgs", "QuantizationModifier", "QuantizationScheme",
    "compute_scale", "dequantize", "fake_quantize", "group_view", "oneshot", "pad_to_group",
    "preset_name_to_scheme", "quantize",
]
