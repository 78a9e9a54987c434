"""What to quantize and how finely: the argument records every stage shares.

API mirror of llmquant/core/scheme.py in the reference (same names, fields and errors).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

#: elements of the reduction axis (K) that share one scale, for weights and activations alike
GROUP_SIZE = 128

_STRATEGIES = ("group", "channel", "token")


@dataclass(frozen=True)
class QuantizationArgs:
    """Symmetric integer quantization of one tensor.

    strategy  "group"   one scale per `group_size` elements of the last axis
              "channel" one scale per weight row, "token" one per activation row
    head_dim  set when the last axis is heads x head_dim (o_proj's input): groups are then
              cut inside each head instead of across two of them
    out_group output rows that share one scale (q/k/v: one scale per output head);
              None keeps a scale per row
    """

    num_bits: int
    strategy: str
    symmetric: bool = True
    dynamic: bool = False
    group_size: Optional[int] = None
    head_dim: Optional[int] = None
    out_group: Optional[int] = None

    def __post_init__(self):
        grouped = self.strategy == "group"
        if grouped and not (self.group_size and self.group_size > 0):
            raise ValueError("strategy='group' requires a positive group_size")
        if not grouped and self.group_size is not None:
            raise ValueError(
                f"group_size is only valid for strategy='group', got {self.strategy!r}"
            )

    @property
    def qmax(self) -> int:
        return (1 << (self.num_bits - 1)) - 1

    @property
    def qmin(self) -> int:
        return -self.qmax - 1


@dataclass(frozen=True)
class QuantizationScheme:
    weights: Optional[QuantizationArgs]
    input_activations: Optional[QuantizationArgs]


def _grouped(bits: int, dynamic: bool) -> QuantizationArgs:
    return QuantizationArgs(num_bits=bits, strategy="group", group_size=GROUP_SIZE, dynamic=dynamic)


# Activations are per token AND per group: a token's scales depend on that token alone, and
# they fall on the weight's group boundaries so the integer GEMM splits into group sums.
PRESET_SCHEMES = {
    f"W{w}A{a}": QuantizationScheme(
        weights=_grouped(w, dynamic=False),
        input_activations=_grouped(a, dynamic=True) if a == 8 else None,
    )
    for w, a in ((4, 8), (8, 8), (4, 16), (8, 16))
}


def preset_name_to_scheme(name: str) -> QuantizationScheme:
    scheme = PRESET_SCHEMES.get(str(name).upper())
    if scheme is None:
        raise ValueError(f"unknown scheme {name!r}, expected one of {list(PRESET_SCHEMES)}")
    return scheme
