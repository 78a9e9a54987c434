"""Padded geometry of one quantized Linear weight, derived in one place.

Mirrors llmquant/core/layout.py: where a head structure sits decides which axis is split
per head and padded -- the output axis for q/k/v (they produce heads), the reduction axis
for o_proj (it consumes them), neither for MLP and lm_head.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional


def round_up(value: int, multiple: int) -> int:
    return (value + multiple - 1) // multiple * multiple


@dataclass(frozen=True)
class WeightLayout:
    out_features: int
    in_features: int
    group_size: int
    in_head_dim: Optional[int] = None   # o_proj
    out_head_dim: Optional[int] = None  # q/k/v_proj

    def __post_init__(self):
        if self.in_head_dim and self.in_features % self.in_head_dim:
            raise ValueError(
                f"in_features {self.in_features} is not a multiple of head_dim {self.in_head_dim}"
            )
        if self.out_head_dim and self.out_features % self.out_head_dim:
            raise ValueError(
                f"out_features {self.out_features} is not a multiple of head_dim {self.out_head_dim}"
            )

    def _padded(self, size: int, head_dim: Optional[int]) -> int:
        if head_dim:
            return size // head_dim * round_up(head_dim, self.group_size)
        return round_up(size, self.group_size)

    @property
    def padded_in(self) -> int:
        return self._padded(self.in_features, self.in_head_dim)

    @property
    def padded_out(self) -> int:
        return self._padded(self.out_features, self.out_head_dim)

    @property
    def in_groups(self) -> int:
        return self.padded_in // self.group_size

    @property
    def scale_rows(self) -> int:
        """One scale row per output head when heads sit on the output axis, else per row."""
        return self.out_features // self.out_head_dim if self.out_head_dim else self.out_features

    @property
    def num_scales(self) -> int:
        return self.scale_rows * self.in_groups

    @property
    def stored_elements(self) -> int:
        return self.padded_out * self.padded_in

    def weight_bytes(self, num_bits: int) -> int:
        return self.stored_elements * num_bits // 8

    def bits_per_real_element(self, num_bits: int, scale_bytes: int) -> float:
        """Storage bits per weight that carries data, so padding shows up in the number."""
        stored_bits = 8 * (self.weight_bytes(num_bits) + self.num_scales * scale_bytes)
        return stored_bits / (self.out_features * self.in_features)


def layout_for(out_features: int, in_features: int, args, group_size=None) -> WeightLayout:
    return WeightLayout(
        out_features=out_features,
        in_features=in_features,
        group_size=group_size or args.group_size,
        in_head_dim=args.head_dim,
        out_head_dim=args.out_group,
    )
