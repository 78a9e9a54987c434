"""Nibble packing for 4-bit codes (llmquant/packing/packing.py).

A 4-bit code c in [-8, 7] is stored as the unsigned nibble c + 8. Two share a byte: the
even index in the low nibble, the odd one in the high nibble, so (-3, 5) -> (5, 13) -> 0xD5.
int8 codes are stored as they are. The GEMV kernel reads exactly these bytes.
"""

from __future__ import annotations

import torch

INT4_BIAS = 8
INT4_MIN, INT4_MAX = -8, 7


def pack_int4(values: torch.Tensor) -> torch.Tensor:
    """[..., n] int8 codes in [-8, 7] -> [..., n / 2] uint8; n must be even."""
    n = values.shape[-1]
    if n % 2:
        raise ValueError(f"last dim {n} must be even to pack into nibbles")
    if values.numel():
        lo_v, hi_v = int(values.min()), int(values.max())
        if lo_v < INT4_MIN or hi_v > INT4_MAX:
            raise ValueError(f"values must be in [{INT4_MIN}, {INT4_MAX}], got [{lo_v}, {hi_v}]")
    nibbles = (values.to(torch.int16) + INT4_BIAS).to(torch.uint8).unflatten(-1, (n // 2, 2))
    return (nibbles[..., 0] | (nibbles[..., 1] << 4)).contiguous()


def unpack_int4(packed: torch.Tensor) -> torch.Tensor:
    """[..., n / 2] uint8 -> [..., n] int8, undoing pack_int4."""
    pair = torch.stack((packed & 0x0F, packed >> 4), dim=-1).to(torch.int16) - INT4_BIAS
    return pair.flatten(-2).to(torch.int8)


def pack_weight(qweight: torch.Tensor, num_bits: int) -> torch.Tensor:
    if num_bits == 4:
        return pack_int4(qweight)
    if num_bits == 8:
        return qweight.contiguous()
    raise ValueError(f"unsupported num_bits {num_bits}, expected 4 or 8")


def unpack_weight(stored: torch.Tensor, num_bits: int) -> torch.Tensor:
    if num_bits == 4:
        return unpack_int4(stored)
    if num_bits == 8:
        return stored.to(torch.int8)
    raise ValueError(f"unsupported num_bits {num_bits}, expected 4 or 8")
