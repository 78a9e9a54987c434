"""What a model costs as it stands: the four numbers a result row carries beside its timings
(llmquant/eval/run.py:119-125, definitions of llmquant/core/metrics.py:103-200).

  deployed_bytes          on disk: codes at their bit width + fp32 scales (canonical padding included),
                          everything else as bf16; an untied, quantized lm_head is counted beside the
                          embedding table it no longer shares
  decode_bytes_per_token  what one decoded token reads: every Linear and lm_head in full, norms, the routed
                          fraction of stacked experts; the embedding is a row lookup and is not counted
  bits_per_element        weight bits plus amortized scale bits per REAL weight element, parameter-weighted
  kv_bytes_per_token      keys and values of one token of context over all layers and kv heads, one fp32
                          scale per token per head when quantized

The reference computes them on the bf16 model from the recipe; here they are read off the model as
deployed (the quantized modules know what they store), which gives the same numbers for the same recipe.
"""

from __future__ import annotations

import torch.nn as nn

SCALE_BYTES = 4
BF16_BYTES = 2
GB = 1024 ** 3


def kv_cache_bytes_per_token(model, num_bits: int | None) -> int:
    config = model.config
    kv_heads = getattr(config, "num_key_value_heads", None) or config.num_attention_heads
    head_dim = getattr(config, "head_dim", None) or config.hidden_size // config.num_attention_heads
    elements = 2 * config.num_hidden_layers * kv_heads * head_dim
    if num_bits is None:
        return elements * BF16_BYTES
    return elements * num_bits // 8 + 2 * config.num_hidden_layers * kv_heads * SCALE_BYTES


def deployed_cost(model, kv_cache_bits: int | None = None) -> dict:
    from llmquant.quantizers.experts import _QuantExperts
    from llmquant.quantizers.kernel import KernelQuantLinear
    from llmquant.quantizers.real import RealQuantLinear

    embed = model.get_input_embeddings()
    config = getattr(model, "config", None)
    total, live = getattr(config, "num_local_experts", None), getattr(config, "num_experts_per_tok", None)
    routed = live / total if total and live else 1.0
    disk = decode = 0
    bits = elements = 0.0
    owned = set()

    def stored(module):
        """(bytes, real elements) of a quantized or plain Linear."""
        if isinstance(module, KernelQuantLinear):
            nbytes = module.qdata.numel() * module.qdata.element_size() + module.wscale.numel() * SCALE_BYTES
            return nbytes, module.out_features * module.in_features
        if isinstance(module, RealQuantLinear):
            num_bits = module.scheme.weights.num_bits
            return module.qweight.numel() * num_bits // 8 + module.wscale.numel() * SCALE_BYTES, module.qweight.numel()
        return module.weight.numel() * BF16_BYTES, module.weight.numel()

    for name, module in model.named_modules():
        if isinstance(module, (KernelQuantLinear, RealQuantLinear, nn.Linear)):
            nbytes, real = stored(module)
            disk += nbytes
            decode += nbytes
            bits += nbytes * 8
            elements += real
            owned.update(id(t) for t in list(module.parameters(recurse=False)) + list(module.buffers(recurse=False)))
        elif isinstance(module, _QuantExperts):
            tensors = list(module.buffers(recurse=False))
            nbytes = sum(t.numel() * t.element_size() for t in tensors)
            disk += nbytes
            decode += int(nbytes * routed)
            bits += nbytes * 8
            elements += module.num_experts * 3 * module.hidden_dim * module.intermediate_dim
            owned.update(id(t) for t in tensors)
    # (a tied lm_head was walked as a Linear above and owns the shared tensor: counted once, read in full)
    for p in model.parameters():
        if id(p) in owned:
            continue
        nbytes = p.numel() * BF16_BYTES
        disk += nbytes
        if p is not embed.weight:
            decode += nbytes  # norms: tiny, but read every token
    return {"deployed_bytes": int(disk), "decode_bytes_per_token": int(decode),
            "bits_per_element": bits / max(elements, 1.0),
            "kv_bytes_per_token": kv_cache_bytes_per_token(model, kv_cache_bits)}


def cost_columns(cost: dict) -> dict:
    """The four columns run_one adds to a row (llmquant/eval/run.py:119-125)."""
    return {"kv_gb_per_1k_context": cost["kv_bytes_per_token"] * 1024 / GB,
            "size_gb": cost["deployed_bytes"] / GB,
            "decode_gb_per_token": cost["decode_bytes_per_token"] / GB,
            "bits_per_element": cost["bits_per_element"]}
