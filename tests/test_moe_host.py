"""Mixture-of-Experts host logic on the CPU: the routing plan, the modifier's handling of stacked
expert weights, and the real-mode block against the oracle (reference tests/test_moe.py)."""

import numpy as np
import pytest
import torch
import torch.nn as nn

import llmq_oracle as oracle
from conftest import rel_l2, to_np
from llmquant import QuantConfig, oneshot
from llmquant.core.scheme import QuantizationScheme
from llmquant.core.modifier import stacked_expert_blocks, stacked_expert_parameters
from llmquant.quantizers import RealQuantExperts, quant_experts_for, quantize_expert_stack, route_plan


def mixtral_config(**kw):
    from transformers import MixtralConfig

    base = dict(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=8,
                num_key_value_heads=4, vocab_size=1000, num_local_experts=4, num_experts_per_tok=2,
                max_position_embeddings=512)
    base.update(kw)
    return MixtralConfig(**base)


def mixtral_model(**kw):
    from transformers import MixtralForCausalLM

    torch.manual_seed(0)
    return MixtralForCausalLM(mixtral_config(**kw)).to(torch.bfloat16).eval()


def expert_block(experts=8, hidden=256, inter=128, top_k=4):
    from transformers.models.mixtral.modeling_mixtral import MixtralExperts

    cfg = mixtral_config(hidden_size=hidden, intermediate_size=inter, num_local_experts=experts,
                         num_experts_per_tok=top_k, num_hidden_layers=1, num_key_value_heads=8)
    torch.manual_seed(0)
    block = MixtralExperts(cfg).to(torch.bfloat16).eval()
    with torch.no_grad():
        block.gate_up_proj.normal_(0, 0.02)
        block.down_proj.normal_(0, 0.02)
    return block, cfg


def routing(tokens, experts, top_k, seed=0):
    gen = torch.Generator().manual_seed(seed)
    index = torch.stack([torch.randperm(experts, generator=gen)[:top_k] for _ in range(tokens)])
    return index, torch.rand(tokens, top_k, generator=gen).to(torch.bfloat16)


@pytest.mark.parametrize("tokens,experts,top_k,limit", [(1, 8, 4, 8), (6, 8, 4, 8), (6, 4, 2, 2), (9, 3, 3, 4), (5, 64, 8, 8)])
def test_route_plan_covers_every_row_once_and_never_straddles(tokens, experts, top_k, limit):
    index, _ = routing(tokens, experts, top_k, seed=tokens)
    order, (block_expert, block_row0, block_rows) = route_plan(index, experts, limit)
    want_order, (we, w0, wr) = oracle.route_plan(index.numpy(), experts, limit)
    assert order.tolist() == want_order.tolist()
    assert block_expert.tolist() == we.tolist() and block_row0.tolist() == w0.tolist()
    assert block_rows.tolist() == wr.tolist()
    assert block_expert.dtype == block_row0.dtype == block_rows.dtype == torch.int32
    expert_of_row = index.reshape(-1)[order]
    covered = []
    for e, r0, n in zip(block_expert.tolist(), block_row0.tolist(), block_rows.tolist()):
        assert 0 <= n <= limit
        if n:
            assert (expert_of_row[r0:r0 + n] == e).all()
            covered.extend(range(r0, r0 + n))
    assert sorted(covered) == list(range(index.numel()))
    assert len(block_expert) == experts * max(1, -(-index.numel() // limit))  # shape from shapes only


def test_quantize_expert_stack_is_per_expert_weight_quantization():
    block, _ = expert_block(experts=3)
    args = QuantConfig(mlp_weight="int4").scheme("mlp_weight").weights
    codes, scales = quantize_expert_stack(block.gate_up_proj.data, args)
    assert codes.shape == (3, 256, 2, 128) and codes.dtype == torch.int8 and scales.shape == (3, 256, 2)
    for e in range(3):
        want_q, want_s = oracle.canonical_weight(to_np(block.gate_up_proj.data[e]), 4, 128)
        assert np.array_equal(codes[e].numpy(), want_q) and np.array_equal(scales[e].numpy(), want_s)


@pytest.mark.parametrize("bits", ["int8", "int4"])
def test_real_experts_match_the_oracle_and_track_bf16(bits):
    block, cfg = expert_block()
    scheme = QuantConfig(mlp_weight=bits).scheme("mlp_weight")
    real = RealQuantExperts.from_experts(block, scheme)
    hidden = torch.randn(5, cfg.hidden_size, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
    index, weights = routing(5, cfg.num_local_experts, cfg.num_experts_per_tok, seed=2)
    with torch.no_grad():
        got = real(hidden, index, weights)
        dense = block(hidden, index, weights)
    want = oracle.moe_experts_real(to_np(hidden), index.numpy(), to_np(weights), real.qgate_up.numpy(),
                                   real.sgate_up.numpy(), real.qdown.numpy(), real.sdown.numpy())
    assert rel_l2(to_np(got), want) <= 1e-2
    assert (got.float() - dense.float()).abs().max() < dense.float().abs().max() * (0.1 if bits == "int8" else 0.5)


@pytest.mark.parametrize("mode,expected", [("fake", "MixtralExperts"), ("real", "RealQuantExperts")])
def test_each_mode_puts_the_right_module_in_the_moe_block(mode, expected):
    model = mixtral_model()
    gate_before = model.model.layers[0].mlp.gate.weight.data.clone()
    experts_before = model.model.layers[0].mlp.experts.gate_up_proj.data.clone()
    oneshot(model, QuantConfig(attn_weight="int8", mlp_weight="int8", head_weight="int8").to_modifier(mode=mode))
    block = model.model.layers[0].mlp.experts
    assert type(block).__name__ == expected
    assert torch.equal(model.model.layers[0].mlp.gate.weight.data, gate_before)  # the router is never quantized
    if mode == "fake":
        after = block.gate_up_proj.data
        assert after.shape == experts_before.shape and not torch.equal(after, experts_before)
        want = oracle.fake_quantize(to_np(experts_before), 8, "bf16", "group", 128)
        assert np.array_equal(to_np(after), want)
    ids = torch.randint(0, 1000, (1, 12), generator=torch.Generator().manual_seed(3))
    with torch.no_grad():
        assert torch.isfinite(model(ids).logits).all()


def test_experts_lookup_and_structure_checks():
    assert quant_experts_for("fake") is None
    assert quant_experts_for("real") is RealQuantExperts
    with pytest.raises(ValueError, match="unsupported mode"):
        quant_experts_for("bogus")
    model = mixtral_model()
    names = [n for n, _ in stacked_expert_parameters(model)]
    assert "model.layers.0.mlp.experts.gate_up_proj" in names and "model.layers.1.mlp.experts.down_proj" in names
    assert [n for n, _ in stacked_expert_blocks(model)] == ["model.layers.0.mlp.experts", "model.layers.1.mlp.experts"]

    class Strange(nn.Module):
        def __init__(self):
            super().__init__()
            self.gate_up_proj = nn.Parameter(torch.zeros(4, 512, 256))  # no down_proj, no act_fn

    odd = nn.Module()
    odd.layers = nn.ModuleList([nn.Module()])
    odd.layers[0].mlp = nn.Module()
    odd.layers[0].mlp.experts = Strange()
    with pytest.raises(NotImplementedError, match="missing"):
        stacked_expert_blocks(odd)
    with pytest.raises(ValueError, match="needs a weight scheme"):
        RealQuantExperts.from_experts(expert_block()[0], QuantizationScheme(weights=None, input_activations=None))
