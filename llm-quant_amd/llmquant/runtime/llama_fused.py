"""The decode step as five launches per layer.

LlamaKernelRuntime walks a decoder layer the way transformers does, one PyTorch kernel per
elementwise operation: about 40 launches per layer, 670 per token, and at 3-4 us each the
launches, not the weights, set the token rate. Here the same arithmetic, with the same
rounding points, is folded into the kernels that have to run anyway:

  1  RMSNorm -> q|k|v projection          (one GEMV over the concatenated weight)
  2  RoPE -> KV quantize-append -> attention   (one kernel, one workgroup per kv head)
  3  o_proj (+ head padding of its input) -> + residual
  4  RMSNorm -> gate|up projection         (one GEMV over the concatenated weight)
  5  SiLU(gate) * up -> down_proj -> + residual

plus embedding lookup, final RMSNorm -> lm_head, and argmax. Prefill is unchanged
(LlamaKernelRuntime's): it is one call over many tokens and its cost is in the GEMMs.

Requirements on the model (met by oneshot(..., mode="kernel") of a Llama architecture with
QuantConfig's defaults): every Linear a KernelQuantLinear with group size 128 and no bias,
q/k/v sharing bit width and out_group, gate/up sharing bit width.
"""

from __future__ import annotations

import torch

from llmquant.hip.build import load_extension
from llmquant.quantizers.kernel import KernelQuantLinear
from llmquant.runtime.llama_decode import LlamaKernelRuntime

PRO_NONE, PRO_RMSNORM, PRO_SILU_MUL, PRO_ATTN_MERGE = 0, 1, 2, 3


def _fusable(*mods) -> bool:
    first = mods[0]
    for m in mods:
        if not isinstance(m, KernelQuantLinear) or m.bias is not None or m._int8_act:
            return False
        if m.qdata.dtype != first.qdata.dtype or m.out_group != first.out_group:
            return False
        if m.qdata.shape[1:] != first.qdata.shape[1:] or m.scheme.weights.group_size != 128:
            return False
        if m.qdata.shape[1] % 4:  # the matrix-core GEMV walks a row four groups at a time
            return False
    return True


# Cached tokens from which a grouped-query model's decode step runs its attention launch with 16 splits, and with 32 (a
# cache of 2048 rows or more takes the matrix-core form of the launch from 8 splits on). Measured on the 1B architecture
# in a 32 K-row cache, us a token by cached tokens, for 8 / 16 / 32 splits: 600: 560 / 576 / 615; 1000: 551 / - / -;
# 2000: 562 / 576 / 615; 3500: 574 / 577 / 616; 7000: - / 601 / 616; 15000: - / 646 / 644; 31000: - / 732 / 706
# (the vector-ALU form, which caches below 2048 rows keep, with 8 splits: 546-551 / 555 / 578 / 595 at 600 / 1000 / 2000 /
# 3500, 673 at 7000)
MID_CONTEXT_FROM = 5120
LONG_CONTEXT_FROM = 16384


def _code_bits(qdata) -> int:
    return 4 if qdata.dtype == torch.uint8 else 8


class PreparedRows:
    """Normed rows of a prompt in the tiled fused GEMM's prepared form (operand order, per-group sums) inside that
    GEMM's workspace, in place of the tensor: what llmq_add_rmsnorm_prepared leaves."""

    def __init__(self, workspace, rows, dtype):
        self.workspace, self.rows, self.dtype = workspace, rows, dtype


class _Fused:
    """Concatenated storage of Linears that read the same activation."""

    def __init__(self, *mods):
        self.qdata = torch.cat([m.qdata for m in mods], dim=0).contiguous()
        self.wscale = torch.cat([m.wscale for m in mods], dim=0).contiguous()
        self.out_group = mods[0].out_group
        self.sources = _sources(mods)


def _sources(mods):
    """What a concatenation was built from: the buffers' addresses and versions (a buffer that was
    replaced or written in place since makes the copy stale)."""
    return tuple((t.data_ptr(), t._version, tuple(t.shape)) for m in mods for t in (m.qdata, m.wscale))


def _fused(owner, name, *mods):
    """The concatenation of `mods`, kept on `owner` (the attention / MLP module) between runtimes: a
    generate call builds a new runtime, and copying 0.4 GB of weights again each time is a
    millisecond of its time to first token."""
    kept = owner.__dict__.get(name)
    if kept is None or kept.sources != _sources(mods):
        kept = _Fused(*mods)
        owner.__dict__[name] = kept
    return kept


class LlamaFusedRuntime(LlamaKernelRuntime):
    def __init__(self, model, max_len: int, kv_bits: int = 8, exact_prefill: bool = False, attn_splits=None):
        """attn_splits: workgroups per query head in the attention launch. None picks enough to put
        a workgroup on every CU (and more for long caches); 1 keeps each head in one workgroup and
        hands o_proj a finished attention output instead of partial records."""
        super().__init__(model, max_len, kv_bits, exact_prefill)
        self._ext = load_extension()
        # A cache of many thousand rows is often mostly empty: the split count (and with it the kernel form) a step
        # runs with follows the tokens the cache holds, through regimes [(from this many cached tokens, splits)] with
        # a captured step each.
        self.regimes = None          # None: one regime, attn_splits
        if attn_splits is None:
            # one workgroup per CU at least; grouped-query models on long caches: 16 splits from 5120 cached tokens and
            # 32 from 16384 (the kernel takes the four query heads of a kv head together with the cache's codes as
            # matrix-core operands); others: four more splits per 2048 rows of cache up to 16
            grouped = self.kv_heads > 0 and (self.q_heads // self.kv_heads) % 4 == 0
            short = max(1, 256 // max(self.q_heads, 1))
            if grouped and short < 16 and max_len > MID_CONTEXT_FROM:
                self.regimes = [(0, short), (MID_CONTEXT_FROM, 16)]
                if max_len > LONG_CONTEXT_FROM:
                    self.regimes.append((LONG_CONTEXT_FROM, 32))
                attn_splits = self.regimes[-1][1]
            elif grouped and short < 16:
                attn_splits = short
            elif grouped and max_len >= 12288:
                attn_splits = 32
            else:
                attn_splits = max(short, min(16, (max_len + 2047) // 2048 * 4))
        if kv_bits == 16:
            # an unquantized cache of the model's dtype (the kv_cache=bf16 ablation under this runtime): only the
            # split attention launch reads it, one regime
            if self.dtype not in (torch.bfloat16, torch.float16):
                raise ValueError("an unquantized cache needs a bfloat16 or float16 model")
            self.regimes = None
            attn_splits = max(2, min(int(attn_splits), 16))
        self.attn_splits = int(attn_splits)
        self._splits_now = self.attn_splits
        self._graphs = {}            # split count -> (graph, logits, next_token)
        self._partials = torch.zeros(self._ext.kv_attend_partials_floats(self.q_heads, self.head_dim,
                                                                         max([self.attn_splits] + [c for _, c in self.regimes or []])),
                                     dtype=torch.float32, device=self.device) if self.attn_splits > 1 else None
        self.fused_layers = []
        for layer in self.layers:
            attn, mlp = layer.self_attn, layer.mlp
            if not (_fusable(attn.q_proj, attn.k_proj, attn.v_proj) and _fusable(mlp.gate_proj, mlp.up_proj)
                    and _fusable(attn.o_proj) and _fusable(mlp.down_proj)):
                raise ValueError("the fused decode step needs kernel-mode Linears (group 128, a multiple of 4 groups per "
                                 "row, no bias, weight-only) with q/k/v and gate/up sharing a bit width")
            for name in ("q_proj", "k_proj", "v_proj"):
                proj = getattr(attn, name)
                if proj.out_group and proj.qdata.shape[0] % proj.out_group:
                    raise ValueError(f"{name} rows are not a whole number of scale tiles: the concatenated "
                                     "q|k|v weight would misalign the scale rows of what follows it")
            if any(m.out_group for m in (mlp.gate_proj, mlp.up_proj, mlp.down_proj)):
                raise ValueError("the fused decode step takes MLP weights with one scale row per output row "
                                 "(out_group 0)")
            args = attn.o_proj.scheme.weights
            self.fused_layers.append(dict(
                qkv=_fused(attn, "_llmq_fused_qkv", attn.q_proj, attn.k_proj, attn.v_proj),
                gate_up=_fused(mlp, "_llmq_fused_gate_up", mlp.gate_proj, mlp.up_proj),
                o=attn.o_proj, down=mlp.down_proj,
                o_head_dim=args.head_dim if attn.o_proj._needs_padding else 0,
                # act(gate) * up inside the gate|up launch: a row tile there is eight gate rows and their up rows
                act_in_gate_up=mlp.gate_proj.qdata.shape[0] % 8 == 0,
                norm1=layer.input_layernorm.weight.detach().contiguous(), eps1=layer.input_layernorm.variance_epsilon,
                norm2=layer.post_attention_layernorm.weight.detach().contiguous(),
                eps2=layer.post_attention_layernorm.variance_epsilon))
        head = model.lm_head
        if not _fusable(head):
            raise ValueError("the fused decode step needs a kernel-mode lm_head")
        self._init_token_pick(model, head.qdata.shape[0])

    def _init_token_pick(self, model, head_rows: int):
        """The final norm's weight and what the token pick at the end of a step needs."""
        self.final_norm = model.model.norm.weight.detach().contiguous()
        self.final_eps = model.model.norm.variance_epsilon
        # The launch that picks a step's token also looks up that token's embedding for the next step
        # (llmq_argmax_advance_embed), so a step starts at its first GEMV. Plain nn.Embedding tables of the
        # model's dtype only; anything else keeps the embedding module's own launch.
        table = model.model.embed_tokens
        # (and of the logits' dtype, which is the model's: _forward and _step must take the same branch)
        plain = (type(table) is torch.nn.Embedding and table.max_norm is None and table.weight.is_contiguous()
                 and table.weight.dtype in (torch.bfloat16, torch.float16, torch.float32)
                 and table.weight.dtype == self.dtype
                 and table.weight.shape[1] % 8 == 0 and table.weight.shape[0] >= head_rows)
        self._embed_table = table.weight.detach() if plain else None
        self._hidden0 = torch.zeros(1, table.weight.shape[1], dtype=table.weight.dtype, device=self.device)
        self._argmax_ws = torch.zeros(self._ext.argmax_workspace_ints(), dtype=torch.int32, device=self.device)

    # ---- the prompt pass: q|k|v and gate|up as one projection each ----------------------------------
    def _takes_tile(self, rows, dtype, fused, prepared=False):
        """Whether _project sends this many rows of this dtype to the tiled fused GEMM (`prepared`: when the norm in
        front of it can write them in the GEMM's prepared form, which saves the preparation launch)."""
        from llmquant.quantizers.kernel import KERNEL_MAX_ROWS, fused_gemm_takes, tiled_gemm_pays

        n, groups = fused.qdata.shape[0], fused.qdata.shape[1]
        return (dtype in (torch.bfloat16, torch.float16) and rows > KERNEL_MAX_ROWS and not fused_gemm_takes(rows, n, groups)
                and tiled_gemm_pays(rows, n, groups, _code_bits(fused.qdata), prepared))

    def _mlp_in_two_launches(self, rows, dtype, index, layer):
        """Whether _mlp runs this many rows as gate|up with the activation in its store + down_proj."""
        from llmquant.quantizers.kernel import (FUSED_GEMM_MAX_ROWS, TILED_GEMM_MAX_ROWS, dense_branch_cost,
                                                tiled_gemm_cost)

        f = self.fused_layers[index]
        gate_up, down = f["gate_up"], f["down"]
        inter = gate_up.qdata.shape[0] // 2
        # down_proj on rows that the gate|up launch left prepared, against the dense branch behind a SiLU * up launch
        # (6 us) of its own
        down_n, down_groups, down_bits = down.out_features, down.qdata.shape[1], _code_bits(down.qdata)
        down_pays = (tiled_gemm_cost(rows, down_n, down_groups, down_bits, prepared=True)
                     <= 1.05 * (dense_branch_cost(rows, down_n, down_groups, down_bits) + 6.0))
        return (dtype in (torch.bfloat16, torch.float16) and self._one_launch_ops and "SiLU" in type(layer.mlp.act_fn).__name__
                and FUSED_GEMM_MAX_ROWS < rows <= TILED_GEMM_MAX_ROWS and inter % 128 == 0
                and -(-rows // 128) * (inter // 128) >= 160
                and down_pays and down.bias is None and not down._needs_padding and not down._int8_act
                and down.qdata.shape[1] * 128 == inter)

    def _add_norm(self, module, hidden, branch, consumer=None):
        """The base class's, except that rows on their way to a tiled fused GEMM leave the norm in that GEMM's
        prepared form (llmq_add_rmsnorm_prepared: the bits of norm + preparation, one launch and one tensor
        fewer): the second value is then a PreparedRows for _project / _mlp."""
        if (consumer is not None and self._one_launch_ops and hidden.dim() == 2
                and hidden.dtype in (torch.bfloat16, torch.float16)
                and type(module).__name__.endswith("RMSNorm") and hasattr(module, "variance_epsilon")
                and hidden.shape[-1] % 128 == 0 and module.weight.dtype == hidden.dtype
                and (branch is None or branch.dtype == hidden.dtype)):
            kind, index = consumer
            rows, f = hidden.shape[0], self.fused_layers[index]
            fused = f["qkv"] if kind == "qkv" else f["gate_up"]
            direct = isinstance(fused, _Fused) and fused.qdata.shape[1] * 128 == hidden.shape[-1]
            if direct and (self._takes_tile(rows, hidden.dtype, fused, prepared=True)
                           or (kind == "mlp" and self._mlp_in_two_launches(rows, hidden.dtype, index,
                                                                          self.layers[index]))):
                next_n = max(fused.qdata.shape[0], f["down"].out_features if kind == "mlp" else 0)
                hidden, workspace = self._ext.add_rmsnorm_prepared(hidden, branch, module.weight,
                                                                   module.variance_epsilon, next_n)
                return hidden, PreparedRows(workspace, rows, hidden.dtype)
        return super()._add_norm(module, hidden, branch, consumer)

    def _project(self, x, fused):
        """x [tokens, K] times a concatenated weight: what KernelQuantLinear.forward would pick for this
        many rows, once for the whole concatenation (three or two matmuls and dequantize passes fewer
        per layer, and the host's matmul dispatch is the longest part of a prompt pass)."""
        from llmquant.quantizers.kernel import KERNEL_MAX_ROWS, fused_gemm_splits, fused_gemm_takes, tiled_gemm_pays

        if isinstance(x, PreparedRows):   # (_add_norm found that these rows take the tiled GEMM)
            return self._ext.wq_gemm_a16_tile_prepared(x.workspace, x.rows, fused.qdata, fused.wscale, fused.out_group,
                                                       x.dtype)
        rows = x.shape[0]
        if (fused_gemm_takes(rows, fused.qdata.shape[0], fused.qdata.shape[1])
                and x.dtype in (torch.bfloat16, torch.float16)):
            return self._ext.wq_gemm_a16(x, fused.qdata, fused.wscale, fused.out_group,
                                         fused_gemm_splits(rows, fused.qdata.shape[1]))
        if rows <= KERNEL_MAX_ROWS:
            return self._ext.wq_gemv(x, fused.qdata, fused.wscale, fused.out_group)
        if self._takes_tile(rows, x.dtype, fused):
            return self._ext.wq_gemm_a16_tile(x.contiguous(), fused.qdata, fused.wscale, fused.out_group)
        if x.dtype in (torch.bfloat16, torch.float16):
            return self._ext.wq_dense_linear(x.contiguous(), fused.qdata, fused.wscale, fused.out_group, 0)
        return x @ self._ext.dequant_weight(fused.qdata, fused.wscale, fused.out_group, 0, x.dtype).T

    def _qkv(self, index, layer, x):
        out = self._project(x, self.fused_layers[index]["qkv"])
        q_width, kv_width = self.q_heads * self.head_dim, self.kv_heads * self.head_dim
        return out[:, :q_width], out[:, q_width:q_width + kv_width], out[:, q_width + kv_width:]

    def _gate_up(self, index, layer, x):
        out = self._project(x, self.fused_layers[index]["gate_up"])
        half = out.shape[1] // 2
        return out[:, :half], out[:, half:]

    def _mlp(self, index, layer, x):
        """A prompt's MLP in two launches where the shapes allow: the gate|up GEMM's workgroups write
        silu(gate) * up straight into down_proj's prepared activation (the bits of the three launches: the
        condition on the tile count is the one under which the plain gate|up GEMM keeps its reduction axis
        whole as well)."""
        f = self.fused_layers[index]
        gate_up, down = f["gate_up"], f["down"]
        rows = x.rows if isinstance(x, PreparedRows) else x.shape[0]
        if self._mlp_in_two_launches(rows, x.dtype, index, layer):
            if isinstance(x, PreparedRows):
                workspace = self._ext.wq_gemm_a16_tile_gate_up_silu_prepared(x.workspace, rows, gate_up.qdata,
                                                                             gate_up.wscale, gate_up.out_group,
                                                                             down.out_features, x.dtype)
            else:
                workspace = self._ext.wq_gemm_a16_tile_gate_up_silu(x.contiguous(), gate_up.qdata, gate_up.wscale,
                                                                    gate_up.out_group, down.out_features)
            return self._ext.wq_gemm_a16_tile_prepared(workspace, rows, down.qdata, down.wscale, down.out_group, x.dtype)
        return super()._mlp(index, layer, x)

    def _forward(self, token_ids, cos, sin, decode: bool):
        if not decode:
            return super()._forward(token_ids, cos, sin, decode)
        ext, cache, splits = self._ext, self.cache, self._splits_now
        # (the row _set_step_inputs or the previous step's token pick left for this token)
        hidden = self._hidden0 if self._embed_table is not None else self.model.model.embed_tokens(token_ids)
        for index, f in enumerate(self.fused_layers):
            qkv = ext.wq_gemv_fused(hidden, f["qkv"].qdata, f["qkv"].wscale, f["qkv"].out_group, PRO_RMSNORM,
                                    f["norm1"], f["eps1"], 0, None)
            if splits > 1:
                # partial records per (head, split), merged by o_proj while it stages its activation
                ext.kv_rope_append_attend_split(qkv, self.cos_table, self.sin_table, cache.k_codes[index],
                                                cache.v_codes[index], cache.k_scale[index], cache.v_scale[index],
                                                self._partials, cache.position, self.scaling, self.q_heads,
                                                splits)
                hidden = ext.wq_gemv_attn_merge(self._partials, splits, self.head_dim, f["o"].qdata,
                                                f["o"].wscale, f["o"].out_group, f["o_head_dim"], hidden,
                                                hidden.dtype)
            else:
                ctx = ext.kv_rope_append_attend(qkv, self.cos_table, self.sin_table, cache.k_codes[index],
                                                cache.v_codes[index], cache.k_scale[index], cache.v_scale[index],
                                                cache.position, self.scaling, self.q_heads)
                hidden = ext.wq_gemv_fused(ctx, f["o"].qdata, f["o"].wscale, f["o"].out_group, PRO_NONE, None, 0.0,
                                           f["o_head_dim"], hidden)
            if f["act_in_gate_up"]:
                act = ext.wq_gemv_gate_up_silu(hidden, f["gate_up"].qdata, f["gate_up"].wscale, PRO_RMSNORM,
                                               f["norm2"], f["eps2"])
                hidden = ext.wq_gemv_fused(act, f["down"].qdata, f["down"].wscale, 0, PRO_NONE, None, 0.0, 0, hidden)
            else:
                gate_up = ext.wq_gemv_fused(hidden, f["gate_up"].qdata, f["gate_up"].wscale, 0, PRO_RMSNORM,
                                            f["norm2"], f["eps2"], 0, None)
                hidden = ext.wq_gemv_fused(gate_up, f["down"].qdata, f["down"].wscale, 0, PRO_SILU_MUL, None, 0.0,
                                           0, hidden)
        head = self.model.lm_head
        return ext.wq_gemv_fused(hidden, head.qdata, head.wscale, head.out_group, PRO_RMSNORM, self.final_norm,
                                 self.final_eps, 0, None)

    def _splits_for(self, cached_tokens: int) -> int:
        """Split count of the attention launch for a cache that holds this many tokens."""
        if not self.regimes:
            return self.attn_splits
        splits = self.regimes[0][1]
        for start, count in self.regimes:
            if cached_tokens >= start:
                splits = count
        return splits

    def _set_step_inputs(self, token, position: int):
        super()._set_step_inputs(token, position)
        self._splits_now = self._splits_for(position)
        if self._embed_table is not None:
            self._hidden0.copy_(self.model.model.embed_tokens(self.token))

    def _use_graph_of(self, splits: int) -> bool:
        kept = self._graphs.get(splits)
        if kept is None:
            return False
        self.graph, self.logits, self.next_token = kept
        self._splits_now = splits
        return True

    @torch.no_grad()
    def capture(self, token, position: int):
        """One captured step per regime: the one `position` falls in is captured (or, if it has been, made current)."""
        if self._use_graph_of(self._splits_for(position)):
            self._set_step_inputs(token, position)
            return
        super().capture(token, position)
        self._graphs[self._splits_now] = (self.graph, self.logits, self.next_token)

    def _ensure_graph(self, token, position: int):
        self.capture(token, position)

    @torch.no_grad()
    def step(self):
        # the cache has grown (or been rewound) into the other regime: its captured step takes over, from the token
        # and position the previous step left on the device
        position = self.cache.get_seq_length()
        if self.regimes and self._splits_for(position) != self._splits_now:
            self.capture(self.token.clone(), position)
        return super().step()

    def _step(self):
        logits = self._forward(self.token, None, None, decode=True)
        # greedy pick, next input token, both position counters and the next step's embedding row in one launch
        if self._embed_table is not None:
            nxt = self._ext.argmax_advance_embed(logits, self.token, self.pos_index, self.cache.position,
                                                 self._embed_table, self._hidden0, self._argmax_ws)
        else:
            nxt = self._ext.argmax_advance(logits, self.token, self.pos_index, self.cache.position)
        return logits, nxt


class LlamaDenseFusedRuntime(LlamaFusedRuntime):
    """The same five-launch decode step for a model whose Linears are plain 16-bit nn.Linear modules, over an
    unquantized cache of the model's dtype (kv_bits 16): the baseline's runtime. The reference times the
    bf16 model and the quantized one under one runtime (llmquant/eval/verify.py:44-47); this is what makes
    that possible here, where the quantized side's runtime is the fused step. Launch for launch it is
    LlamaFusedRuntime's step with llmq_dense_gemv_fused in place of the quantized GEMVs; the prompt pass is the
    walk's, with the library's matmuls over the concatenated weights."""

    def __init__(self, model, max_len: int, kv_bits: int = 16, exact_prefill: bool = False, attn_splits=None):
        if kv_bits != 16:
            raise ValueError("the 16-bit baseline's fused step runs over an unquantized cache (kv_bits 16)")
        LlamaKernelRuntime.__init__(self, model, max_len, 16, exact_prefill)
        if self.dtype not in (torch.bfloat16, torch.float16):
            raise ValueError("the dense fused decode step takes bfloat16 or float16 models")
        self._ext = load_extension()
        self.regimes = None
        # (the o_proj launch merges split-attention records: at least two splits)
        self.attn_splits = int(attn_splits or max(2, 256 // max(self.q_heads, 1)))
        self._splits_now = self.attn_splits
        self._graphs = {}
        self._partials = torch.zeros(self._ext.kv_attend_partials_floats(self.q_heads, self.head_dim, self.attn_splits),
                                     dtype=torch.float32, device=self.device)

        def plain(*mods):
            return all(type(m) is torch.nn.Linear and m.bias is None and m.weight.dtype == self.dtype
                       and m.weight.shape[1] % 8 == 0 for m in mods)

        self.fused_layers = []
        for layer in self.layers:
            attn, mlp = layer.self_attn, layer.mlp
            if not plain(attn.q_proj, attn.k_proj, attn.v_proj, attn.o_proj, mlp.gate_proj, mlp.up_proj, mlp.down_proj):
                raise ValueError("the dense fused decode step needs plain 16-bit nn.Linear modules without bias")
            if "SiLU" not in type(mlp.act_fn).__name__:
                raise ValueError("the dense fused decode step computes SiLU(gate) * up")
            cat = lambda *mods: torch.cat([m.weight.detach() for m in mods], dim=0).contiguous()
            self.fused_layers.append(dict(
                qkv=cat(attn.q_proj, attn.k_proj, attn.v_proj), gate_up=cat(mlp.gate_proj, mlp.up_proj),
                o=attn.o_proj.weight.detach().contiguous(), down=mlp.down_proj.weight.detach().contiguous(),
                inter=mlp.gate_proj.weight.shape[0],
                norm1=layer.input_layernorm.weight.detach().contiguous(), eps1=layer.input_layernorm.variance_epsilon,
                norm2=layer.post_attention_layernorm.weight.detach().contiguous(),
                eps2=layer.post_attention_layernorm.variance_epsilon))
        if not plain(model.lm_head):
            raise ValueError("the dense fused decode step needs a plain 16-bit lm_head")
        self.head_weight = model.lm_head.weight.detach().contiguous()
        self._init_token_pick(model, self.head_weight.shape[0])

    # the prompt pass: the library's matmuls, q|k|v and gate|up over the concatenated weights
    def _qkv(self, index, layer, x):
        out = x @ self.fused_layers[index]["qkv"].T
        q_width, kv_width = self.q_heads * self.head_dim, self.kv_heads * self.head_dim
        return out[:, :q_width], out[:, q_width:q_width + kv_width], out[:, q_width + kv_width:]

    def _gate_up(self, index, layer, x):
        out = x @ self.fused_layers[index]["gate_up"].T
        half = out.shape[1] // 2
        return out[:, :half], out[:, half:]

    def _mlp(self, index, layer, x):
        return LlamaKernelRuntime._mlp(self, index, layer, x)

    def _forward(self, token_ids, cos, sin, decode: bool):
        if not decode:
            return LlamaKernelRuntime._forward(self, token_ids, cos, sin, decode)
        ext, cache, splits = self._ext, self.cache, self._splits_now
        gemv = ext.dense_gemv_fused
        hidden = self._hidden0 if self._embed_table is not None else self.model.model.embed_tokens(token_ids)
        for index, f in enumerate(self.fused_layers):
            qkv = gemv(hidden, f["qkv"], PRO_RMSNORM, f["norm1"], f["eps1"])
            ext.kv_rope_append_attend_split(qkv, self.cos_table, self.sin_table, cache.k_codes[index],
                                            cache.v_codes[index], cache.k_scale[index], cache.v_scale[index],
                                            self._partials, cache.position, self.scaling, self.q_heads, splits)
            hidden = gemv(self._partials, f["o"], PRO_ATTN_MERGE, None, 0.0, hidden, 0, splits, self.head_dim)
            act = gemv(hidden, f["gate_up"], PRO_RMSNORM, f["norm2"], f["eps2"], None, f["inter"])
            hidden = gemv(act, f["down"], PRO_NONE, None, 0.0, hidden)
        return gemv(hidden, self.head_weight, PRO_RMSNORM, self.final_norm, self.final_eps)
