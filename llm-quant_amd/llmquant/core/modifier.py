"""The recipe that rewires a model: which Linear gets which scheme, and the swap itself.

Mirrors llmquant/core/modifier.py. Routing is by module name with the Llama naming the
reference uses, targets are matched by class name, and the quantized module class comes from
the `mode` lookup in llmquant.quantizers.dispatch, imported only when a recipe is applied.
A Mixture-of-Experts block holds its experts as stacked parameters, not Linears: it is found by
parameter name and swapped whole (real, kernel) or quantize-dequantized in place (fake); the
router is left alone, since an error there changes which expert runs rather than a value.
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

# stacked expert weights: transformers 5 gives Mixtral / OLMoE `experts.gate_up_proj`
# [E, 2I, H] and `experts.down_proj` [E, H, I]; w1/w2/w3 are the older per-projection names
MOE_EXPERT_PATTERN = r"re:.*\.experts\.(gate_up_proj|down_proj|w1|w2|w3)$"

SchemeLike = Union[str, QuantizationScheme, None]


def stacked_expert_parameters(model: nn.Module):
    """(name, Parameter) of every stacked expert weight in the model, whatever the recipe."""
    return [(name, p) for name, p in model.named_parameters()
            if p.ndim >= 2 and _name_matches(name, (MOE_EXPERT_PATTERN,))]


def stacked_expert_blocks(model: nn.Module):
    """(name, module) of every module that owns stacked expert weights. Found by structure, not
    class name (OlmoeExperts and MixtralExperts are the same block); one that lacks what the
    quantized block mirrors is refused."""
    blocks = {}
    for name, _ in stacked_expert_parameters(model):
        owner = name.rpartition(".")[0]
        if owner in blocks:
            continue
        module = model.get_submodule(owner)
        missing = [attr for attr in ("gate_up_proj", "down_proj", "act_fn") if not hasattr(module, attr)]
        if missing:
            raise NotImplementedError(
                f"{owner} ({type(module).__name__}) holds stacked expert weights but is missing {missing}; "
                "the quantized expert block mirrors the Mixtral / OLMoE layout (gate_up_proj, down_proj, act_fn)")
        blocks[owner] = module
    return list(blocks.items())


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
        from llmquant.quantizers.dispatch import quant_experts_for, quant_linear_for  # core -> stages, lazily

        quant_cls = quant_linear_for(self.mode)
        experts_cls = quant_experts_for(self.mode)
        self.resolve(model)
        swaps, expert_blocks = [], set()
        if experts_cls is not None and self.mlp_scheme is not None:
            # the experts are the MLP of their layer: they take the mlp scheme
            for name, block in stacked_expert_blocks(model):
                expert_blocks.add(name)
                swaps.append((name, experts_cls.from_experts(block, _as_scheme(self.mlp_scheme))))
        for name, module in model.named_modules():
            if name in expert_blocks or type(module).__name__ not in self.targets:
                continue
            scheme = self.scheme_for(name)
            if scheme is not None:
                swaps.append((name, quant_cls.from_linear(module, scheme)))
        for name, module in swaps:
            _swap_module(model, name, module)
        self._fake_quantize_expert_parameters(model)
        return model

    def expert_parameters(self, model: nn.Module):
        """(name, Parameter) of the stacked expert weights this recipe quantizes."""
        return stacked_expert_parameters(model) if self.mlp_scheme is not None else []

    def _fake_quantize_expert_parameters(self, model: nn.Module) -> None:
        """mode="fake": write quantize-dequantize of each stacked expert weight back into it. The
        other modes have swapped the whole block by now."""
        if self.mode != "fake":
            return
        import torch

        from llmquant.core.quant_ops import fake_quantize

        args = _as_scheme(self.mlp_scheme).weights if self.mlp_scheme is not None else None
        if args is None:
            return
        with torch.no_grad():
            for _, param in self.expert_parameters(model):
                param.copy_(fake_quantize(param.data, args).to(param.dtype))
