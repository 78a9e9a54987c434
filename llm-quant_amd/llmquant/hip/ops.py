"""Python-level ops over the extension (counterpart of llmquant/cuda/ops.py)."""

from __future__ import annotations

import torch

from llmquant.core.observers import pad_to_group
from llmquant.core.scheme import QuantizationArgs
from llmquant.hip.build import load_extension


def _group_size_for(x: torch.Tensor, args: QuantizationArgs) -> int:
    if args.strategy == "group":
        return args.group_size
    if args.strategy in ("channel", "token"):
        return x.shape[-1]  # a single group spanning the row
    raise ValueError(f"unsupported strategy {args.strategy!r}")


def fake_quantize_hip(x: torch.Tensor, args: QuantizationArgs, return_scale: bool = False):
    """Quant-dequant on the GPU, bit-exact with llmquant.core.quant_ops.fake_quantize.

    Groups run along the last axis. A last axis that is not a whole number of groups gets
    the same zero padding the PyTorch form applies, and the padding is trimmed again.
    """
    group_size = _group_size_for(x, args)
    width = x.shape[-1]
    padded = pad_to_group(x, group_size)
    out, scale = load_extension().fake_quant_group(padded, args.num_bits, group_size, return_scale)
    if padded.shape[-1] != width:
        out = out[..., :width]
    return (out, scale) if return_scale else out


def quantize_activation(x: torch.Tensor, args: QuantizationArgs):
    """(int8 codes [..., K], fp32 scales [..., K / group]) for an activation whose last axis
    is already a whole number of groups -- the dynamic A8 quantizer as one kernel."""
    group_size = _group_size_for(x, args)
    return load_extension().quant_group_codes(x, args.num_bits, group_size, False)


# the reference's name for the same op
fake_quantize_cuda = fake_quantize_hip
