"""mode="real": integer weights, arithmetic spelled out group by group in fp32.

Mirrors llmquant/quantizers/real.py. Not a deployment path: it is the module form of the
arithmetic the kernels are compared with, runnable on any device torch supports.
"""

from __future__ import annotations

from contextlib import contextmanager

import torch
import torch.nn as nn

from llmquant.core import observers as obs
from llmquant.core.quant_ops import quantize
from llmquant.core.scheme import QuantizationScheme


@contextmanager
def exact_fp32_matmul():
    """fp32 matmul with TF32 off for the duration, so integer products stay exact."""
    saved = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    try:
        yield
    finally:
        torch.backends.cuda.matmul.allow_tf32 = saved


def quantize_weight(weight: torch.Tensor, args):
    """(int8 codes in the weight's own [out, in] shape, fp32 scales in compute_scale's
    keepdim shape). Padding is applied for the arithmetic and dropped again."""
    scale = obs.compute_scale(weight, args)
    grouped = obs.group_view(weight, args.group_size, args.head_dim)
    if args.out_group:
        tiles = obs.out_block_view(grouped, args.out_group)
        codes = obs.out_unblock(quantize(tiles, scale, args), weight.shape[0])
    else:
        codes = quantize(grouped, scale, args)
    codes = obs.ungroup(codes, weight.shape, args.group_size, args.head_dim)
    return codes.to(torch.int8), scale


class RealQuantLinear(nn.Module):
    """out = sum over groups, in order, of (x_g @ q_g^T) * s_w [* s_x], all in fp32."""

    def __init__(self, qweight, wscale, bias, scheme: QuantizationScheme):
        super().__init__()
        self.register_buffer("qweight", qweight)  # [out, in] int8
        self.register_buffer("wscale", wscale)    # keepdim shape from compute_scale
        self.bias = bias
        self.scheme = scheme
        self.out_features, self.in_features = qweight.shape

    @classmethod
    def from_linear(cls, linear: nn.Linear, scheme: QuantizationScheme):
        if scheme.weights is None:
            raise ValueError("real quant needs a weight scheme; bf16 weights stay nn.Linear")
        codes, scale = quantize_weight(linear.weight.detach(), scheme.weights)
        return cls(codes, scale, linear.bias, scheme)

    def _scale_of_group(self, g: int) -> torch.Tensor:
        """[out_features] weight scales of reduction group g."""
        tile = self.scheme.weights.out_group
        if tile:
            return self.wscale[:, 0, g, 0].repeat_interleave(tile)[: self.out_features]
        return self.wscale[:, g, 0]

    def forward(self, x):
        w_args, a_args = self.scheme.weights, self.scheme.input_activations
        rows = x.reshape(-1, x.shape[-1])
        w_groups = obs.group_view(self.qweight.float(), w_args.group_size, w_args.head_dim)
        if a_args is None:
            a_scale = None
            a_groups = obs.group_view(rows.float(), w_args.group_size, w_args.head_dim)
        else:
            a_scale = obs.compute_scale(rows, a_args)
            a_groups = quantize(obs.group_view(rows, a_args.group_size, a_args.head_dim), a_scale, a_args)

        total = torch.zeros(rows.shape[0], self.out_features, dtype=torch.float32, device=x.device)
        with exact_fp32_matmul():
            for g in range(w_groups.shape[1]):
                term = (a_groups[:, g] @ w_groups[:, g].T) * self._scale_of_group(g)
                if a_scale is not None:
                    term = term * a_scale[:, g]
                total += term
        if self.bias is not None:
            total = total + self.bias.float()
        return total.to(x.dtype).reshape(*x.shape[:-1], self.out_features)

    def extra_repr(self):
        a = self.scheme.input_activations
        return (f"in_features={self.in_features}, out_features={self.out_features}, "
                f"w{self.scheme.weights.num_bits}a{a.num_bits if a else 16}, "
                f"group_size={self.scheme.weights.group_size}")
