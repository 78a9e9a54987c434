"""Quantized stand-ins for a stacked Mixture-of-Experts block (MixtralExperts / OlmoeExperts).

API mirror of RealQuantExperts (llmquant/quantizers/real.py:117-190), KernelQuantExperts and
quantize_expert_stack (llmquant/quantizers/kernel.py:106-289). transformers keeps the experts of
a layer as two stacked parameters, gate_up_proj [E, 2I, H] and down_proj [E, H, I]; both modules
here hold their quantized form, [E, N, groups, group_size] codes and [E, scale_rows, groups] fp32
scales, and are called as `experts(hidden_states, top_k_index, top_k_weights)`.

The kernel module runs every routed expert of a projection in one launch. Which row goes to
which expert is decided on the device (`route_plan`): nothing is read back to the host, so the
block can be recorded into a graph.
"""

from __future__ import annotations

import torch
import torch.nn as nn

from llmquant.core.observers import group_view
from llmquant.core.scheme import QuantizationScheme
from llmquant.packing.packing import pack_int4, unpack_int4
from llmquant.quantizers.real import exact_fp32_matmul, quantize_weight


def quantize_expert_stack(stack: torch.Tensor, args):
    """[E, N, K] float weights -> (codes [E, N, groups, group_size] int8, scales [E, rows, groups] fp32),
    each expert quantized as a Linear weight of its own."""
    codes, scales = [], []
    for weight in stack.detach():
        q, s = quantize_weight(weight, args)
        canonical = group_view(q, args.group_size, args.head_dim).contiguous()
        codes.append(canonical)
        scales.append(s.reshape(-1, canonical.shape[1]).contiguous().float())
    return torch.stack(codes), torch.stack(scales)


def route_plan(top_k_index: torch.Tensor, num_experts: int, limit: int):
    """Sort the (token, slot) rows by expert and cut each expert's run into blocks of at most
    `limit` rows. Returns (order, (block_expert, block_row0, block_rows)): `order[i]` is the flat
    index into top_k_index of the i-th sorted row; block b covers sorted rows block_row0[b] ..
    +block_rows[b]-1, all routed to block_expert[b]. Every expert gets the same number of blocks
    (enough for the case that it takes every row), the unused ones with zero rows, so the shapes
    depend on the input's shape only and no count leaves the device."""
    flat = top_k_index.reshape(-1)
    rows = flat.numel()
    order = torch.argsort(flat, stable=True)
    # a histogram into a buffer of known size: torch.bincount would size its result from the data
    counts = torch.zeros(num_experts, dtype=torch.int64, device=flat.device)
    counts.scatter_add_(0, flat.to(torch.int64), torch.ones_like(flat, dtype=torch.int64))
    first = torch.cumsum(counts, 0) - counts
    per_expert = max(1, -(-rows // limit))
    step = torch.arange(per_expert, device=flat.device, dtype=torch.int64) * limit       # [B]
    expert = torch.arange(num_experts, device=flat.device, dtype=torch.int64)[:, None].expand(-1, per_expert)
    row0 = first[:, None] + step[None, :]
    length = (counts[:, None] - step[None, :]).clamp(0, limit)
    return order, (expert.reshape(-1).int(), row0.reshape(-1).int(), length.reshape(-1).int())


class _QuantExperts(nn.Module):
    """Storage and construction shared by the real and kernel modules."""

    _what = "quantized"

    def __init__(self, qgate_up, sgate_up, qdown, sdown, scheme: QuantizationScheme, hidden_dim: int,
                 intermediate_dim: int, act_fn):
        super().__init__()
        self.scheme = scheme
        self.num_experts = qgate_up.shape[0]
        self.hidden_dim = hidden_dim
        self.intermediate_dim = intermediate_dim
        self.act_fn = act_fn
        self._store(qgate_up, sgate_up, qdown, sdown)

    def _store(self, qgate_up, sgate_up, qdown, sdown):
        self.register_buffer("qgate_up", qgate_up)  # [E, 2I, groups, gs] int8
        self.register_buffer("sgate_up", sgate_up)  # [E, rows, groups] fp32
        self.register_buffer("qdown", qdown)        # [E, H, groups, gs] int8
        self.register_buffer("sdown", sdown)

    @classmethod
    def from_experts(cls, experts: nn.Module, scheme: QuantizationScheme):
        if scheme.weights is None:
            raise ValueError(f"the {cls._what} path needs a weight scheme")
        qgate_up, sgate_up = quantize_expert_stack(experts.gate_up_proj.data, scheme.weights)
        qdown, sdown = quantize_expert_stack(experts.down_proj.data, scheme.weights)
        return cls(qgate_up, sgate_up, qdown, sdown, scheme, hidden_dim=experts.gate_up_proj.shape[2],
                   intermediate_dim=experts.down_proj.shape[2], act_fn=experts.act_fn)

    def _project(self, x, which: str, expert: int):
        raise NotImplementedError

    def _each_hit_expert(self, hidden_states, top_k_index, top_k_weights):
        """MixtralExperts.forward's loop: one expert at a time over the tokens routed to it."""
        final = torch.zeros_like(hidden_states)
        with torch.no_grad():
            mask = nn.functional.one_hot(top_k_index, num_classes=self.num_experts).permute(2, 1, 0)
            hit = torch.greater(mask.sum(dim=(-1, -2)), 0).nonzero()
        for entry in hit:
            expert = int(entry[0])
            if expert == self.num_experts:
                continue
            slot, token = torch.where(mask[expert])
            gate, up = self._project(hidden_states[token], "gate_up", expert).chunk(2, dim=-1)
            out = self._project(self.act_fn(gate) * up, "down", expert)
            out = out * top_k_weights[token, slot, None]
            final.index_add_(0, token, out.to(final.dtype))
        return final

    def extra_repr(self):
        return (f"num_experts={self.num_experts}, hidden={self.hidden_dim}, intermediate={self.intermediate_dim}, "
                f"w{self.scheme.weights.num_bits}, group_size={self.scheme.weights.group_size}")


class RealQuantExperts(_QuantExperts):
    """Integer weights, fp32 matmul per expert: the arithmetic the kernel module is held to."""

    _what = "real"

    def _project(self, x, which, expert):
        codes = getattr(self, f"q{which}")[expert]
        scales = getattr(self, f"s{which}")[expert]
        real_in = self.hidden_dim if which == "gate_up" else self.intermediate_dim
        per_scale = codes.shape[0] // scales.shape[0]
        weight = (codes.float() * scales.repeat_interleave(per_scale, dim=0).unsqueeze(-1)).flatten(1)[:, :real_in]
        with exact_fp32_matmul():
            return (x.float() @ weight.T).to(x.dtype)

    def forward(self, hidden_states, top_k_index, top_k_weights):
        return self._each_hit_expert(hidden_states, top_k_index, top_k_weights)


class KernelQuantExperts(_QuantExperts):
    """Every routed expert of a projection in one launch of the batched GEMV.

    4-bit stacks live in HBM nibble-packed ([E, N, groups, gs/2] uint8, the bytes of the packed
    file); `qgate_up` / `qdown` hand back the canonical int8 view on demand."""

    _what = "kernel"

    def _store(self, qgate_up, sgate_up, qdown, sdown):
        from llmquant.hip.build import load_extension

        bits = self.scheme.weights.num_bits
        pack = (lambda t: t.contiguous() if t.dtype == torch.uint8 else pack_int4(t)) if bits == 4 else (
            lambda t: t.contiguous())
        self.register_buffer("gate_up_data", pack(qgate_up))
        self.register_buffer("sgate_up", sgate_up.contiguous())
        self.register_buffer("down_data", pack(qdown))
        self.register_buffer("sdown", sdown.contiguous())
        self._packed = self.gate_up_data.dtype == torch.uint8
        per_byte = 2 if self._packed else 1
        self._gate_up_padded = self.gate_up_data.shape[2] * self.gate_up_data.shape[3] * per_byte
        self._down_padded = self.down_data.shape[2] * self.down_data.shape[3] * per_byte
        self._weight_args = self.scheme.weights
        self._ext = load_extension()
        # The fused forward folds act_fn(gate) * up into the gate|up launch, which is written for SiLU
        # (MixtralExperts / OlmoeExperts); anything else keeps the operation-by-operation form.
        self._act_is_silu = self._probe_silu()
        self._gemv = self._ext.wq_gemv
        self._gemv_batched = self._ext.wq_gemv_batched
        self._batched_max_rows = self._ext.wq_gemv_batched_max_rows()

    # (the loaded extension is a module object, which copy and pickle refuse: a copy looks it up again)
    def __getstate__(self):
        state = dict(self.__dict__)
        for name in ("_ext", "_gemv", "_gemv_batched"):
            state.pop(name, None)
        return state

    def __setstate__(self, state):
        super().__setstate__(state)
        self._ext = load_extension()
        self._gemv = self._ext.wq_gemv
        self._gemv_batched = self._ext.wq_gemv_batched

    def _probe_silu(self) -> bool:
        probe = torch.linspace(-6.0, 6.0, 25)
        try:
            return bool(torch.equal(self.act_fn(probe), nn.functional.silu(probe)))
        except Exception:
            return False

    @property
    def qgate_up(self) -> torch.Tensor:
        return unpack_int4(self.gate_up_data) if self._packed else self.gate_up_data

    @property
    def qdown(self) -> torch.Tensor:
        return unpack_int4(self.down_data) if self._packed else self.down_data

    # state_dict in the reference's terms: `qgate_up` / `qdown` as int8 [E, N, groups, gs]
    # (llmquant/quantizers/kernel.py:134-137); load_state_dict takes that form or the stored one.
    def _save_to_state_dict(self, destination, prefix, keep_vars):
        super()._save_to_state_dict(destination, prefix, keep_vars)
        kept = {name: destination.pop(prefix + name) for name in ("gate_up_data", "sgate_up", "down_data", "sdown")}
        unpack = unpack_int4 if self._packed else (lambda t: t)
        destination[prefix + "qgate_up"] = unpack(kept["gate_up_data"])
        destination[prefix + "sgate_up"] = kept["sgate_up"]
        destination[prefix + "qdown"] = unpack(kept["down_data"])
        destination[prefix + "sdown"] = kept["sdown"]

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                              error_msgs):
        for theirs, mine in (("qgate_up", "gate_up_data"), ("qdown", "down_data")):
            codes = state_dict.pop(prefix + theirs, None)
            if codes is not None and prefix + mine not in state_dict:
                state_dict[prefix + mine] = pack_int4(codes) if self._packed and codes.dtype == torch.int8 else codes
        super()._load_from_state_dict(state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                                      error_msgs)

    def _stored(self, which):
        if which == "gate_up":
            return self.gate_up_data, self.sgate_up, self.hidden_dim, self._gate_up_padded
        return self.down_data, self.sdown, self.intermediate_dim, self._down_padded

    def _pad(self, x, real_in, padded_in):
        from llmquant.quantizers.kernel import pad_activation

        return pad_activation(x, self._weight_args) if real_in != padded_in else x

    def _matmul(self, x, qweight, wscale, real_in, padded_in):
        """One expert's projection: the GEMV for one or two rows (up to KERNEL_MAX_ROWS for fp32), the fused
        GEMM for FUSED_GEMM_MIN_ROWS .. FUSED_GEMM_MAX_ROWS rows of a 16-bit activation, else dequantize + matmul. `qweight` is that
        expert's slice, stored (packed) or canonical."""
        from llmquant.quantizers.kernel import (FUSED_GEMM_MAX_ROWS, FUSED_GEMM_MIN_ROWS, KERNEL_MAX_ROWS,
                                               fused_gemm_splits)

        x = self._pad(x, real_in, padded_in)
        if qweight.dtype == torch.int8 and self._packed:
            qweight = pack_int4(qweight)
        if (FUSED_GEMM_MIN_ROWS <= x.shape[0] <= FUSED_GEMM_MAX_ROWS and x.dtype in (torch.bfloat16, torch.float16)
                and self._weight_args.group_size == 128):
            return self._ext.wq_gemm_a16(x, qweight.contiguous(), wscale, 0, fused_gemm_splits(x.shape[0], qweight.shape[1]))
        if x.shape[0] <= KERNEL_MAX_ROWS:
            return self._gemv(x, qweight, wscale, 0)
        return x @ self._ext.dequant_weight(qweight.contiguous(), wscale, 0, 0, x.dtype).T

    def _project(self, x, which, expert):
        data, scales, real_in, padded_in = self._stored(which)
        return self._matmul(x, data[expert], scales[expert], real_in, padded_in)

    def _plan(self, top_k_index):
        """`route_plan` in one launch when the sizes fit the kernel's single workgroup (they do wherever the
        batched path runs: a few tokens), else the PyTorch form: the same integers either way."""
        if self._ext.route_plan_supported(top_k_index.numel(), self.num_experts):
            order, *plan = self._ext.route_plan(top_k_index, self.num_experts, self._batched_max_rows)
            return order, tuple(plan)
        return route_plan(top_k_index, self.num_experts, self._batched_max_rows)

    def _batched(self, x, qweight, wscale, plan, real_in, padded_in):
        if qweight.dtype == torch.int8 and self._packed:
            qweight = pack_int4(qweight)
        return self._gemv_batched(self._pad(x, real_in, padded_in), qweight, wscale, *plan, 0)

    def _fusable(self, hidden_states, top_k_index, top_k_weights) -> bool:
        """Whether the four-launch forward applies: SiLU experts, group size 128 with rows of a multiple of
        four groups and no input padding (the matrix-core kernels), a routing problem the plan kernel takes,
        routing weights in the activations' dtype."""
        groups_ok = self.gate_up_data.shape[2] % 4 == 0 and self.down_data.shape[2] % 4 == 0
        return (self._act_is_silu and self._weight_args.group_size == 128 and groups_ok
                and self._gate_up_padded == self.hidden_dim and self._down_padded == self.intermediate_dim
                and self.intermediate_dim % 8 == 0
                and hidden_states.dim() == 2 and hidden_states.is_contiguous()
                and top_k_weights.dtype == hidden_states.dtype and top_k_weights.shape == top_k_index.shape
                and self._ext.route_plan_supported(top_k_index.numel(), self.num_experts))

    def _forward_fused(self, hidden_states, top_k_index, top_k_weights):
        """Plan, gate|up (storing act(gate) * up), down, weighted sum per token: four launches. With one
        token every row reads that token's activation, so `hidden_states[tokens_per_row]` is not formed."""
        ext = self._ext
        tokens, top_k = hidden_states.shape[0], top_k_index.shape[-1]
        rows = top_k_index.numel()
        with torch.no_grad():
            order, *plan = ext.route_plan(top_k_index, self.num_experts, self._batched_max_rows)
        one = tokens == 1
        x = hidden_states if one else hidden_states[order // top_k]
        act = ext.wq_gemv_batched_fused(x, one, rows, self.gate_up_data, self.sgate_up, *plan, True)
        out = ext.wq_gemv_batched_fused(act, False, rows, self.down_data, self.sdown, *plan, False)
        return ext.moe_combine(out, order, top_k_weights.contiguous(), tokens)

    def forward(self, hidden_states, top_k_index, top_k_weights):
        # An expert cannot be picked twice by one token, so no expert sees more rows than there
        # are tokens: the shape alone says whether the batched kernel's run length suffices.
        if hidden_states.shape[0] > self._batched_max_rows:
            return self._each_hit_expert(hidden_states, top_k_index, top_k_weights)
        if self._fusable(hidden_states, top_k_index, top_k_weights):
            return self._forward_fused(hidden_states, top_k_index, top_k_weights)
        return self._forward_unfused(hidden_states, top_k_index, top_k_weights)

    def _forward_unfused(self, hidden_states, top_k_index, top_k_weights):
        """KernelQuantExperts.forward of the reference, operation by operation."""
        top_k = top_k_index.shape[-1]
        with torch.no_grad():
            order, plan = self._plan(top_k_index)
        token, slot = order // top_k, order % top_k
        fused = self._batched(hidden_states[token], self.gate_up_data, self.sgate_up, plan, self.hidden_dim,
                              self._gate_up_padded)
        gate, up = fused.chunk(2, dim=-1)
        out = self._batched(self.act_fn(gate) * up, self.down_data, self.sdown, plan, self.intermediate_dim,
                            self._down_padded)
        out = out * top_k_weights[token, slot, None]
        final = torch.zeros_like(hidden_states)
        final.index_add_(0, token, out.to(final.dtype))
        return final

    def _forward_looped(self, hidden_states, top_k_index, top_k_weights):
        return self._each_hit_expert(hidden_states, top_k_index, top_k_weights)
