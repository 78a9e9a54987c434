"""Cutting the reduction axis into groups, and the abs-max scale of each group.

Mirrors llmquant/core/observers.py of the reference: same functions, same shapes, and the
one arithmetic rule that matters -- the scale is amax divided by qmax with a true fp32
division (a tensor divisor; a Python scalar divisor lowers to a reciprocal multiply and
lands an ulp away from what a kernel computes).
"""

from __future__ import annotations

import torch
import torch.nn.functional as F

from llmquant.core.scheme import QuantizationArgs

SCALE_EPS = 1e-8


def pad_to_group(x: torch.Tensor, group_size: int) -> torch.Tensor:
    """Zero-extend the last axis to the next multiple of `group_size`.

    Zeros cannot raise a symmetric abs-max, so the real elements quantize exactly as they
    would in a group of their own length.
    """
    short = -x.shape[-1] % group_size
    return F.pad(x, (0, short)) if short else x


def group_view(x: torch.Tensor, group_size: int, head_dim: int | None = None) -> torch.Tensor:
    """[..., K] -> [..., groups, group_size], padding a short tail.

    With `head_dim`, K is heads x head_dim and every head is padded to whole groups on its
    own, so no group straddles two heads.
    """
    if head_dim is not None:
        *lead, k = x.shape
        if k % head_dim:
            raise ValueError(f"last dim {k} is not a multiple of head_dim {head_dim}")
        x = x.reshape(*lead, k // head_dim, head_dim)
        return pad_to_group(x, group_size).reshape(*lead, -1, group_size)
    x = pad_to_group(x, group_size)
    return x.unflatten(-1, (x.shape[-1] // group_size, group_size))


def ungroup(y: torch.Tensor, shape, group_size: int, head_dim: int | None = None) -> torch.Tensor:
    """Inverse of group_view for a tensor of original `shape`: flatten, drop the padding."""
    *lead, k = shape
    if head_dim is None:
        return y.reshape(*lead, -1)[..., :k]
    per_head = -(-head_dim // group_size) * group_size
    return y.reshape(*lead, k // head_dim, per_head)[..., :head_dim].reshape(*lead, k)


def out_block_view(x: torch.Tensor, out_group: int) -> torch.Tensor:
    """[out, ...] -> [tiles, out_group, ...]: rows of a tile will share one scale."""
    short = -x.shape[0] % out_group
    if short:
        x = F.pad(x, [0, 0] * (x.dim() - 1) + [0, short])
    return x.reshape(-1, out_group, *x.shape[1:])


def out_unblock(y: torch.Tensor, out: int) -> torch.Tensor:
    return y.flatten(0, 1)[:out]


def compute_scale(x: torch.Tensor, args: QuantizationArgs) -> torch.Tensor:
    """fp32 abs-max / qmax, floored at SCALE_EPS, with the reduced axis kept for broadcast."""
    values = x.float()
    if args.strategy == "group":
        grouped = group_view(values, args.group_size, args.head_dim)
        if args.out_group:
            amax = out_block_view(grouped, args.out_group).abs().amax(dim=(1, -1), keepdim=True)
        else:
            amax = grouped.abs().amax(dim=-1, keepdim=True)
    elif args.strategy in ("channel", "token"):
        amax = values.abs().amax(dim=-1, keepdim=True)
    else:
        raise ValueError(f"unsupported strategy {args.strategy!r}")
    qmax = torch.tensor(float(2 ** (args.num_bits - 1) - 1), dtype=torch.float32, device=amax.device)
    return torch.clamp(amax / qmax, min=SCALE_EPS)
