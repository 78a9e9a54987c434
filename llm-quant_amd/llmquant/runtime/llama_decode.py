"""A decode runtime for Llama-architecture models on the kernel path.

The reference drives a quantized model through HF `model(...)` / `generate`
(llmquant/runtime/graph_decode.py:75-131), which with a quantized cache means ~20 PyTorch
kernels of cache quantization per layer per token and no graph capture. This runtime walks
the same modules itself -- same operations, same order, same rounding points as
transformers' LlamaDecoderLayer (RMSNorm in fp32 then cast, RoPE and residuals in the model
dtype, SiLU*up in the model dtype) -- but reads and writes the integer KV cache with the
append / decode-attention kernels, so one token is a fixed launch sequence with every
changing quantity (token id, position, length) on the device. That sequence is captured once
and replayed.

Linears are whatever the model holds: KernelQuantLinear after oneshot(mode="kernel"), or
plain nn.Linear for a bf16 model.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F

from llmquant.hip.build import load_extension
from llmquant.runtime.kv_cache import KernelQuantCache

WARMUP_CALLS = 3


def _rotate_half(x):
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


class LlamaKernelRuntime:
    """Prefill + greedy decode of one sequence over a LlamaForCausalLM-shaped model."""

    # Prompts of up to this many tokens (by head_dim) go through the package's own attention kernel, which is
    # built for the short walk (every CU busy at 512 tokens, where it takes under half the library's time) and
    # level with the library's flash kernel at these lengths; between them and 8192 tokens the library is 5-10 %
    # ahead.
    PROMPT_ATTENTION_MAX_TOKENS = {64: 2048, 128: 1536}

    def __init__(self, model, max_len: int, kv_bits: int = 8, exact_prefill: bool = False):
        cfg = model.config
        self.exact_prefill = exact_prefill
        self.model = model
        self.device = next(model.parameters()).device
        self.dtype = next(model.parameters()).dtype
        self.layers = list(model.model.layers)
        self.q_heads = cfg.num_attention_heads
        self.kv_heads = cfg.num_key_value_heads
        self.head_dim = getattr(cfg, "head_dim", None) or cfg.hidden_size // cfg.num_attention_heads
        self.scaling = self.head_dim ** -0.5
        self.max_len = max_len
        self._ext = load_extension()
        # RMSNorm, RoPE and SiLU * up as one launch each (16-bit models); False walks the PyTorch modules
        self._one_launch_ops = self.dtype in (torch.bfloat16, torch.float16)
        self.cache = KernelQuantCache(len(self.layers), self.kv_heads, self.head_dim, max_len, kv_bits,
                                      q_heads=self.q_heads, device=self.device,
                                      **({"dtype": self.dtype} if kv_bits == 16 else {}))
        # cos / sin for every position, computed the way LlamaRotaryEmbedding.forward does
        # (fp32 outer product, cat, cos/sin, attention_scaling, cast) so lookups equal recomputation
        rope = model.model.rotary_emb
        positions = torch.arange(max_len, device=self.device, dtype=torch.float32)
        freqs = torch.outer(positions, rope.inv_freq.to(self.device, torch.float32))
        emb = torch.cat((freqs, freqs), dim=-1)
        scale = getattr(rope, "attention_scaling", 1.0)
        self.cos_table = (emb.cos() * scale).to(self.dtype)
        self.sin_table = (emb.sin() * scale).to(self.dtype)
        # device-side state of the captured step
        self.token = torch.zeros(1, dtype=torch.long, device=self.device)
        self.pos_index = torch.zeros(1, dtype=torch.long, device=self.device)
        self.graph = None
        self.logits = None
        self.next_token = None

    # ---- shared pieces -----------------------------------------------------------------------------
    def _rope(self, q, k, cos, sin):
        """q [T, Hq, D], k [T, Hkv, D]; cos/sin [T, D]. transformers' apply_rotary_pos_emb."""
        cos, sin = cos[:, None, :], sin[:, None, :]
        return (q * cos) + (_rotate_half(q) * sin), (k * cos) + (_rotate_half(k) * sin)

    def _fp32_causal_attention(self, q, k, v):
        """softmax(q k^T) v with everything in fp32 and one rounding at the end: the arithmetic
        the decode kernel uses, for prompts (q [T, Hq, D]; k, v [Hkv, T, D])."""
        tokens, rep = q.shape[0], self.q_heads // self.kv_heads
        qf = q.float().transpose(0, 1).reshape(self.kv_heads, rep, tokens, self.head_dim)
        scores = torch.matmul(qf, k.float()[:, None].transpose(-1, -2)) * self.scaling
        causal = torch.ones(tokens, tokens, dtype=torch.bool, device=q.device).tril()
        probs = torch.softmax(scores.masked_fill(~causal, float("-inf")), dim=-1)
        ctx = torch.matmul(probs, v.float()[:, None])  # [Hkv, rep, T, D]
        return ctx.reshape(self.q_heads, tokens, self.head_dim).transpose(0, 1).reshape(tokens, -1).to(q.dtype)

    # ---- the elementwise pieces, one launch each where the module is the stock Llama one -----------
    def _norm(self, module, x):
        """LlamaRMSNorm in one launch (seven PyTorch kernels otherwise)."""
        if (self._one_launch_ops and type(module).__name__.endswith("RMSNorm") and hasattr(module, "variance_epsilon")
                and x.shape[-1] % 8 == 0 and module.weight.dtype == x.dtype):
            return self._ext.rmsnorm(x, module.weight, module.variance_epsilon)
        return module(x)

    def _add_norm(self, module, hidden, branch, consumer=None):
        """(hidden + branch, norm(hidden + branch)): the residual add in the launch of the norm after it.
        branch None: (hidden, norm(hidden)). `consumer`: ("qkv" | "mlp", layer index) when the normed rows go
        to that projection of a prompt pass and nowhere else (a runtime may then hand them over in another form)."""
        if branch is None:
            return hidden, self._norm(module, hidden)
        if (self._one_launch_ops and type(module).__name__.endswith("RMSNorm") and hasattr(module, "variance_epsilon")
                and hidden.shape[-1] % 8 == 0 and module.weight.dtype == hidden.dtype and branch.dtype == hidden.dtype):
            return self._ext.add_rmsnorm(hidden, branch, module.weight, module.variance_epsilon)
        hidden = hidden + branch
        return hidden, module(hidden)

    def _rotated(self, q, k, cos, sin):
        """q [T, Hq*D], k [T, Hkv*D] -> rotated [T, Hq, D], [T, Hkv, D]."""
        tokens = q.shape[0]
        if self._one_launch_ops and self.head_dim % 16 == 0 and q.dtype == cos.dtype:
            return self._ext.rope_qk(q, k, cos, sin, self.q_heads, self.kv_heads)
        return self._rope(q.view(tokens, self.q_heads, self.head_dim), k.view(tokens, self.kv_heads, self.head_dim),
                          cos, sin)

    def _rope_append_in_one_launch(self, q, k, v, cos):
        """RoPE and the cache append of a prompt as one launch (llmq_rope_kv_append): stock rotation,
        heads of 64 or 128, rows of the projections with a contiguous last axis."""
        return (self._one_launch_ops and self.cache.num_bits != 16 and self.head_dim in (64, 128)
                and q.dtype == cos.dtype and cos.is_contiguous()
                and all(t.dim() == 2 and t.stride(1) == 1 for t in (q, k, v)))

    def _qkv(self, index, layer, x):
        """The three projections of a layer, each [tokens, heads * head_dim]."""
        attn = layer.self_attn
        return attn.q_proj(x), attn.k_proj(x), attn.v_proj(x)

    def _gate_up(self, index, layer, x):
        return layer.mlp.gate_proj(x), layer.mlp.up_proj(x)

    def _gated(self, index, layer, x):
        mlp = layer.mlp
        gate, up = self._gate_up(index, layer, x)
        packets = (gate.shape[-1] % 8 == 0 and gate.stride(-1) == 1 and up.stride(-1) == 1
                   and gate.data_ptr() % 16 == 0 and up.data_ptr() % 16 == 0
                   and (gate.dim() != 2 or (gate.stride(0) % 8 == 0 and up.stride(0) % 8 == 0)))
        if self._one_launch_ops and "SiLU" in type(mlp.act_fn).__name__ and packets:
            return self._ext.silu_mul(gate, up)
        return mlp.act_fn(gate) * up

    def _mlp(self, index, layer, x):
        """down_proj(act_fn(gate_proj(x)) * up_proj(x))."""
        return layer.mlp.down_proj(self._gated(index, layer, x))

    def _layer(self, index, layer, hidden, cos, sin, decode: bool, branch=None, defer: bool = False):
        """One decoder layer. `branch`: the previous layer's MLP output, still to be added to `hidden`
        (done in the launch of this layer's first norm). `defer`: hand back (hidden, MLP output) and
        leave the last add to the caller's next norm; otherwise the layer's output."""
        attn = layer.self_attn
        tokens = hidden.shape[0]
        hidden, x = self._add_norm(layer.input_layernorm, hidden, branch, None if decode else ("qkv", index))
        q, k, v = self._qkv(index, layer, x)
        k_dq = v_dq = None
        if not decode and self._rope_append_in_one_launch(q, k, v, cos):
            cache = self.cache
            q, k_dq, v_dq = self._ext.rope_kv_append(q, k, v, cos, sin, cache.k_codes[index], cache.v_codes[index],
                                                     cache.k_scale[index], cache.v_scale[index], cache.position,
                                                     self.q_heads, True)
        else:
            if v.stride(0) != self.kv_heads * self.head_dim:
                v = v.contiguous()  # the append wants k's strides, and k comes out of the rotation contiguous
            v = v.view(tokens, self.kv_heads, self.head_dim)
            q, k = self._rotated(q, k, cos, sin)
            appended = self.cache.append(index, k.transpose(0, 1), v.transpose(0, 1), return_dequantized=not decode)
            if not decode:
                k_dq, v_dq = appended
        if decode:
            ctx = self.cache.attend(index, q[0].contiguous(), self.scaling).reshape(1, -1)
        elif self.exact_prefill:
            # prompt: attention sees the fake-quantized K/V of the prompt itself, which is what
            # FakeQuantCache.update returns on an empty cache
            ctx = self._fp32_causal_attention(q, k_dq, v_dq)
        elif (self._one_launch_ops and tokens <= self.PROMPT_ATTENTION_MAX_TOKENS.get(self.head_dim, 0)
              and q.dim() == 3 and q.is_contiguous() and k_dq.is_contiguous() and v_dq.is_contiguous()):
            # the same causal grouped-query softmax(q k^T) v as the library call below, walked by four waves
            # per 32 queries, and written as [tokens, heads * head_dim] directly
            ctx = self._ext.prefill_attention(q, k_dq, v_dq, self.scaling)
        else:
            ctx = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k_dq[None], v_dq[None],
                                                 is_causal=True, scale=self.scaling, enable_gqa=True)
            ctx = ctx[0].transpose(0, 1).reshape(tokens, -1)
        hidden, x = self._add_norm(layer.post_attention_layernorm, hidden, attn.o_proj(ctx),
                                   None if decode else ("mlp", index))
        out = self._mlp(index, layer, x)
        return (hidden, out) if defer else hidden + out

    def _forward(self, token_ids, cos, sin, decode: bool):
        hidden, branch = self.model.model.embed_tokens(token_ids), None
        for index, layer in enumerate(self.layers):
            hidden, branch = self._layer(index, layer, hidden, cos, sin, decode, branch, defer=True)
        # only the last position goes on: its residual add and the final norm in one launch
        _, last = self._add_norm(self.model.model.norm, hidden[-1:].contiguous(),
                                 None if branch is None else branch[-1:].contiguous())
        return self.model.lm_head(last)

    # ---- prefill ------------------------------------------------------------------------------------
    @torch.no_grad()
    def prefill(self, input_ids):
        """Run the prompt (cache must be empty), return the first generated token [1]."""
        ids = input_ids.reshape(-1).to(self.device)
        tokens = ids.shape[0]
        if tokens + 1 > self.max_len:
            raise ValueError(f"prompt of {tokens} tokens does not fit a cache of {self.max_len}")
        self.cache.set_position(0)
        self.cache.length.fill_(tokens)
        logits = self._forward(ids, self.cos_table[:tokens], self.sin_table[:tokens], decode=False)
        self.cache.set_position(tokens)
        # (one row of logits: the kernel that the decode step uses, first maximum like torch.argmax)
        return self._ext.argmax_row(logits) if logits.shape[0] == 1 and logits.is_contiguous() else logits.argmax(-1)

    # ---- decode ---------------------------------------------------------------------------------------
    def _step(self):
        """One token: reads self.token / self.pos_index / cache.position, leaves logits and the
        argmax, and advances every device-side counter for the next call."""
        self.cache.length.copy_(self.cache.position + 1)
        cos = self.cos_table.index_select(0, self.pos_index)
        sin = self.sin_table.index_select(0, self.pos_index)
        logits = self._forward(self.token, cos, sin, decode=True)
        nxt = logits.argmax(-1)
        self.token.copy_(nxt)
        self.pos_index.add_(1)
        self.cache.position.add_(1)
        return logits, nxt

    def _set_step_inputs(self, token, position: int):
        self.token.copy_(token.reshape(1))
        self.pos_index.fill_(position)
        self.cache.set_position(position)

    @torch.no_grad()
    def capture(self, token, position: int):
        """Warm up on a side stream, capture one step, and rewind: the warmup and capture runs
        write cache slots position.. which the first replays overwrite with the same values."""
        self._set_step_inputs(token, position)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(WARMUP_CALLS):
                self._set_step_inputs(token, position)
                self._step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self._set_step_inputs(token, position)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.logits, self.next_token = self._step()
        self._set_step_inputs(token, position)

    def _ensure_graph(self, token, position: int):
        """A captured step that starts from (token, position): captured now, or, on a kept runtime, the one it has
        (it reads token and position from the device)."""
        if self.graph is None:
            self.capture(token, position)
        else:
            self._set_step_inputs(token, position)

    @torch.no_grad()
    def step(self):
        """Replay one step; the token fed is the previous step's argmax, already on the device."""
        self.graph.replay()
        self.cache._host_length += 1
        return self.next_token

    @torch.no_grad()
    def eager_step(self, token, position: int):
        self._set_step_inputs(token, position)
        logits, nxt = self._step()
        self.cache._host_length = position + 1
        return logits, nxt

    @torch.no_grad()
    def generate(self, input_ids, max_new_tokens: int, use_graph: bool = True):
        """Greedy generation; returns the full sequence [1, prompt + new] like model.generate."""
        ids = input_ids.reshape(1, -1).to(self.device)
        prompt = ids.shape[1]
        if prompt + max_new_tokens > self.max_len:
            raise ValueError("prompt + new tokens exceed the cache")
        nxt = self.prefill(ids)
        out = [nxt.reshape(1, 1)]
        if max_new_tokens > 1:
            if use_graph:
                self._ensure_graph(nxt, prompt)
                for _ in range(max_new_tokens - 1):
                    out.append(self.step().clone().reshape(1, 1))
            else:
                for i in range(max_new_tokens - 1):
                    _, nxt = self.eager_step(nxt, prompt + i)
                    out.append(nxt.clone().reshape(1, 1))
        return torch.cat([ids, *out], dim=1)
