"""The recipe that rewires a model: which Linear gets which scheme, and the swap itself.

Mirrors llmquant/core/modifier.py (dense models; the stacked-expert MoE path is not part of
this build). Routing is by module name with the Llama naming the reference uses, targets
are matched by class name, and the quantized module class comes from the `mode` lookup in
llmquant.quantizers.dispatch, imported only when a recipe is applied.
"""

from __future__ import annotations

import re
from dataclasses import dataclass, replace
from typing import Optional, Tuple, Union

import torch.nn as nn

from llmquant.core.scheme import QuantizationScheme, preset_name_to_scheme

ATTN_PATTERN = r"re:.*\.self_attn\..*_proj$"
MLP_PATTERN = r"re:.*\.mlp\..*_proj$"
# the one Linear whose INPUT is heads x head_dim
O_PROJ_PATTERN = r"re:.*\.self_attn\.o_proj$"
# Linears whose OUTPUT is heads x head_dim, a fused qkv included
QKV_PATTERN = r"re:.*\.self_attn\.(q|k|v|qkv)_proj$"

SchemeLike = Union[str, QuantizationScheme, None]


def _as_scheme(value: SchemeLike) -> Optional[QuantizationScheme]:
    if value is None or isinstance(value, QuantizationScheme):
        return value
    return preset_name_to_scheme(value)


def _name_matches(name: str, patterns) -> bool:
    for pattern in patterns:
        if pattern.startswith("re:"):
            if re.match(pattern[3:], name):
                return True
        elif pattern == name:
            return True
    return False


def _swap_module(model: nn.Module, dotted: str, new: nn.Module) -> None:
    owner, _, leaf = dotted.rpartition(".")
    setattr(model.get_submodule(owner) if owner else model, leaf, new)


@dataclass
class QuantizationModifier:
    scheme: SchemeLike = None                 # default for targeted Linears
    targets: Tuple[str, ...] = ("Linear",)
    ignore: Tuple[str, ...] = ("lm_head",)
    lm_head_scheme: SchemeLike = None         # None keeps lm_head in bf16
    mode: str = "fake"
    attn_scheme: SchemeLike = None            # overrides `scheme` under self_attn
    mlp_scheme: SchemeLike = None             # overrides `scheme` under mlp
    kv_cache_bits: Optional[int] = None       # resolved bit width, None = bf16 cache
    head_dim: Optional[int] = None            # read off the model by resolve()
    qkv_out_scale_per_head: bool = True       # q/k/v: one scale per output head

    def resolve(self, model) -> "QuantizationModifier":
        """Pick up head_dim from model.config unless it was given."""
        cfg = getattr(model, "config", None)
        if cfg is not None and self.head_dim is None:
            hd = getattr(cfg, "head_dim", None)
            if hd is None and getattr(cfg, "num_attention_heads", None):
                hd = cfg.hidden_size // cfg.num_attention_heads
            self.head_dim = hd
        return self

    def _head_aware(self, scheme):
        # heads on the reduction axis: both operands must be cut on the same boundaries
        if scheme is None or not self.head_dim:
            return scheme
        w, a = scheme.weights, scheme.input_activations
        return QuantizationScheme(
            weights=replace(w, head_dim=self.head_dim) if w else None,
            input_activations=replace(a, head_dim=self.head_dim) if a else None,
        )

    def _out_head_aware(self, scheme):
        # heads on the output axis: only the weight has one
        if scheme is None or not self.head_dim or scheme.weights is None:
            return scheme
        return QuantizationScheme(
            weights=replace(scheme.weights, out_group=self.head_dim),
            input_activations=scheme.input_activations,
        )

    def scheme_for(self, name: str) -> Optional[QuantizationScheme]:
        """The scheme for the Linear called `name`; None leaves it alone."""
        if name == "lm_head":
            return _as_scheme(self.lm_head_scheme)
        if _name_matches(name, self.ignore):
            return None
        if self.attn_scheme is not None and _name_matches(name, (ATTN_PATTERN,)):
            scheme = _as_scheme(self.attn_scheme)
            if _name_matches(name, (O_PROJ_PATTERN,)):
                return self._head_aware(scheme)
            if self.qkv_out_scale_per_head and _name_matches(name, (QKV_PATTERN,)):
                return self._out_head_aware(scheme)
            return scheme
        if self.mlp_scheme is not None and _name_matches(name, (MLP_PATTERN,)):
            return _as_scheme(self.mlp_scheme)
        return _as_scheme(self.scheme)

    def apply(self, model: nn.Module) -> nn.Module:
        from llmquant.quantizers.dispatch import quant_linear_for  # core -> stages, lazily

        quant_cls = quant_linear_for(self.mode)
        self.resolve(model)
        swaps = []
        for name, module in model.named_modules():
            if type(module).__name__ not in self.targets:
                continue
            scheme = self.scheme_for(name)
            if scheme is not None:
                swaps.append((name, quant_cls.from_linear(module, scheme)))
        for name, module in swaps:
            _swap_module(model, name, module)
        return model
