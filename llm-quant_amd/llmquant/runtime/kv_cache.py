"""The quantized KV cache as real integers in HBM.

FakeQuantCache (llmquant/quantizers/fake.py:39-55) quantizes K and V on write and then stores
the dequantized bf16 values; the accounting the reference reports for it (17 KB per cached
token at int8 instead of 32 KB) is for a cache that keeps the codes. This is that cache:
static-shaped per layer ([kv_heads, t_max, head_dim] codes + [kv_heads, t_max] fp32 scales),
written by the append kernel at a position that lives on the device and read back inside the
decode-attention kernel. Nothing about it changes shape or address from step to step, so a
decode step that uses it can be captured in a HIP graph -- which the reference's
quantized cache cannot (llmquant/runtime/graph_decode.py:40-43).
"""

from __future__ import annotations

import torch

from llmquant.hip.build import load_extension


class KernelQuantCache:
    """K/V codes and scales for every layer of one sequence (batch 1).

    num_bits   8 (int8 codes) or 4 (nibble-packed); 16: an unquantized cache of `dtype` values (the 16-bit
               baseline run through the same decode step; only the fused step's attention launch reads it)
    position   device int32 [1]: where the next token is written
    length     device int32 [1]: tokens valid for attention (position + tokens being added)
    """

    def __init__(self, num_layers: int, kv_heads: int, head_dim: int, max_len: int, num_bits: int = 8,
                 q_heads: int | None = None, device="cuda", dtype=torch.bfloat16):
        if num_bits not in (4, 8, 16):
            raise ValueError(f"KV cache bits must be 4 or 8 (or 16 for an unquantized cache), got {num_bits}")
        if num_bits == 16 and dtype not in (torch.bfloat16, torch.float16):
            raise ValueError("an unquantized cache holds bfloat16 or float16 values")
        self.num_bits, self.num_layers = num_bits, num_layers
        self.kv_heads, self.head_dim, self.max_len = kv_heads, head_dim, max_len
        self._ext = load_extension()
        width = head_dim // 2 if num_bits == 4 else head_dim
        code_dtype = {8: torch.int8, 4: torch.uint8, 16: dtype}[num_bits]
        shape = (num_layers, kv_heads, max_len, width)
        self.k_codes = torch.zeros(shape, dtype=code_dtype, device=device)
        self.v_codes = torch.zeros(shape, dtype=code_dtype, device=device)
        fill = torch.ones if num_bits == 16 else torch.zeros
        self.k_scale = fill(num_layers, kv_heads, max_len, dtype=torch.float32, device=device)
        self.v_scale = fill(num_layers, kv_heads, max_len, dtype=torch.float32, device=device)
        self.position = torch.zeros(1, dtype=torch.int32, device=device)
        self.length = torch.zeros(1, dtype=torch.int32, device=device)
        q_heads = q_heads or kv_heads
        # one workspace per layer: launches that share one must not overlap, and layers of a
        # captured step could in principle be reordered onto other streams by a caller
        floats = self._ext.kv_decode_workspace_floats(q_heads, head_dim, max_len)
        self.workspace = torch.zeros(num_layers, floats, dtype=torch.float32, device=device)
        self._host_length = 0  # mirror for prefill bookkeeping only; decode never reads it

    # ---- bookkeeping ------------------------------------------------------------------------------
    def get_seq_length(self) -> int:
        return self._host_length

    def set_position(self, position: int) -> None:
        """Next write position (host call; inside a graph the tensors are advanced instead)."""
        self._host_length = position
        self.position.fill_(position)
        self.length.fill_(position)

    def advance(self, tokens: int = 1) -> None:
        """Move the write position forward on the device (capturable)."""
        self.position.add_(tokens)
        self._host_length += tokens

    def bytes_per_token(self) -> int:
        """Codes + scales stored per cached token over all layers, K and V."""
        if self.num_bits == 16:
            return 2 * self.num_layers * self.kv_heads * self.head_dim * 2
        width = self.head_dim if self.num_bits == 8 else self.head_dim // 2
        return 2 * self.num_layers * self.kv_heads * (width + 4)

    # ---- per-layer operations ------------------------------------------------------------------------
    def append(self, layer: int, key: torch.Tensor, value: torch.Tensor, return_dequantized: bool = False):
        """key / value: [kv_heads, n_new, head_dim] (any strides with a contiguous last axis).
        Writes at position .. position + n_new - 1. With return_dequantized, hands back what
        FakeQuantCache.update would have returned for these tokens."""
        if self.num_bits == 16:
            # the unquantized cache: a copy at the host-side position (prompt passes only; the fused decode step
            # appends inside its attention launch)
            start, stop = self._host_length, self._host_length + key.shape[1]
            self.k_codes[layer][:, start:stop] = key
            self.v_codes[layer][:, start:stop] = value
            return (key.contiguous(), value.contiguous()) if return_dequantized else (None, None)
        return self._ext.kv_append(key, value, self.k_codes[layer], self.v_codes[layer], self.k_scale[layer],
                                   self.v_scale[layer], self.position, return_dequantized)

    def attend(self, layer: int, query: torch.Tensor, scaling: float) -> torch.Tensor:
        """query [q_heads, head_dim] -> [q_heads, head_dim], over tokens 0 .. length - 1."""
        return self._ext.kv_decode_attention(query, self.k_codes[layer], self.v_codes[layer], self.k_scale[layer],
                                             self.v_scale[layer], self.workspace[layer], self.length, scaling)

    def dequantized(self, layer: int, n_tokens: int, dtype=torch.bfloat16):
        """(keys, values) [kv_heads, n_tokens, head_dim] as the fake-quant cache would hold them."""
        k = self._ext.kv_dequant(self.k_codes[layer], self.k_scale[layer], n_tokens, dtype)
        v = self._ext.kv_dequant(self.v_codes[layer], self.v_scale[layer], n_tokens, dtype)
        return k, v


def make_kernel_cache_factory(num_bits, model, max_len: int):
    """Counterpart of make_cache_factory (llmquant/quantizers/fake.py:58-62) for the kernel
    path: a zero-argument factory of KernelQuantCache sized for `model`, or None for bf16."""
    if num_bits is None:
        return None
    cfg = model.config
    head_dim = getattr(cfg, "head_dim", None) or cfg.hidden_size // cfg.num_attention_heads
    device = next(model.parameters()).device
    return lambda: KernelQuantCache(cfg.num_hidden_layers, cfg.num_key_value_heads, head_dim, max_len, num_bits,
                                    q_heads=cfg.num_attention_heads, device=device)
