"""Quantize, dequantize, and the two chained -- the PyTorch statement of the arithmetic.

Mirrors llmquant/core/quant_ops.py. The HIP op in llmquant.hip matches fake_quantize bit
for bit; this module is the slow, portable form of the same thing and runs anywhere.
"""

from __future__ import annotations

import torch

from llmquant.core import observers as obs
from llmquant.core.scheme import QuantizationArgs


def quantize(x: torch.Tensor, scale: torch.Tensor, args: QuantizationArgs) -> torch.Tensor:
    """Integer-valued fp32 codes: divide, round half to even (torch.round), clamp.

    Elementwise; for a grouped scheme pass `x` already in its group_view.
    """
    top = 2 ** (args.num_bits - 1) - 1
    return torch.round(x.float() / scale).clamp_(-top - 1, top)


def dequantize(q: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    return q * scale


def fake_quantize(x: torch.Tensor, args: QuantizationArgs) -> torch.Tensor:
    """Quantize then dequantize, returned in x's dtype and shape."""
    scale = obs.compute_scale(x, args)
    if args.strategy != "group":
        return dequantize(quantize(x, scale, args), scale).to(x.dtype)
    grouped = obs.group_view(x, args.group_size, args.head_dim)
    if args.out_group:
        tiles = obs.out_block_view(grouped, args.out_group)
        values = obs.out_unblock(dequantize(quantize(tiles, scale, args), scale), x.shape[0])
    else:
        values = dequantize(quantize(grouped, scale, args), scale)
    return obs.ungroup(values, x.shape, args.group_size, args.head_dim).to(x.dtype)
