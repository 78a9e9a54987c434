"""The batched expert GEMV and the kernel-mode Mixture-of-Experts block on the GPU
(reference tests/test_moe.py:283-399)."""

import numpy as np
import pytest
import torch

import llmq_oracle as oracle
from conftest import rel_l2, to_np
from test_moe_host import expert_block, mixtral_model, routing

from llmquant import QuantConfig, oneshot

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ext():
    from llmquant.hip import load_extension

    return load_extension()


def kernel_block(bits="int8", **kw):
    """hidden and intermediate 512: four groups of 128, the smallest rows the matrix-core kernels
    take (shorter ones go to the fallback kernels, whose summation order is another)."""
    from llmquant.quantizers import KernelQuantExperts, RealQuantExperts

    kw.setdefault("hidden", 512)
    kw.setdefault("inter", 512)
    block, cfg = expert_block(**kw)
    block = block.cuda()
    scheme = QuantConfig(mlp_weight=bits).scheme("mlp_weight")
    return block, KernelQuantExperts.from_experts(block, scheme).cuda().eval(), \
        RealQuantExperts.from_experts(block, scheme).cuda().eval(), cfg


@pytest.mark.parametrize("bits", ["int8", "int4"])
@pytest.mark.parametrize("tokens", [1, 4, 8])
def test_the_batched_kernel_is_bit_exact_per_row_against_single_launches(ext, bits, tokens):
    _, quant, _, cfg = kernel_block(bits)
    torch.manual_seed(tokens)
    hidden = torch.randn(tokens, cfg.hidden_size, device="cuda", dtype=torch.bfloat16)
    index, _ = routing(tokens, cfg.num_local_experts, cfg.num_experts_per_tok, seed=tokens)
    index = index.cuda()
    with torch.no_grad():
        order, plan = quant._plan(index)
        rows = hidden[order // cfg.num_experts_per_tok]
        batched = quant._batched(rows, quant.gate_up_data, quant.sgate_up, plan, quant.hidden_dim, quant._gate_up_padded)
        flat = index.reshape(-1)
        looped = torch.empty_like(batched)
        for expert in flat.unique().tolist():
            sel = (flat[order] == expert).nonzero().flatten()
            for r in sel.tolist():  # one row per launch: the single-row kernel is the yardstick
                looped[r] = ext.wq_gemv(rows[r:r + 1], quant.gate_up_data[expert], quant.sgate_up[expert], 0)[0]
    assert torch.equal(batched, looped)
    assert all(part.is_cuda for part in plan) and order.is_cuda  # nothing came back to the host


@pytest.mark.parametrize("bits", [8, 4])
def test_runs_of_every_length_and_entries_that_must_be_ignored(ext, bits):
    """The op on a hand-made plan: runs of 1..8 rows, an empty entry, an entry pointing past the
    rows and one naming an expert that does not exist (both ignored, their rows left zero)."""
    gen = torch.Generator().manual_seed(0)
    experts, n, k = 5, 96, 512
    w = (torch.randn(experts, n, k, generator=gen) * 0.02).to(torch.bfloat16)
    stacks = [oracle.canonical_weight(to_np(w[e]), bits, 128) for e in range(experts)]
    codes = np.stack([c for c, _ in stacks])
    q = torch.from_numpy(oracle.pack_int4(codes) if bits == 4 else codes).cuda()
    s = torch.from_numpy(np.stack([sc for _, sc in stacks])).cuda()
    lengths = [1, 2, 3, 4, 5, 6, 7, 8]
    rows = sum(lengths) + 3
    x = torch.randn(rows, k, generator=gen).to(torch.bfloat16).cuda()
    block_expert = [i % experts for i in range(len(lengths))] + [2, 1, 7]
    block_row0 = list(np.cumsum([0] + lengths[:-1])) + [0, rows - 2, 0]
    block_rows = lengths + [0, 5, 2]  # empty; runs past the last row; no such expert
    plan = [torch.tensor(v, dtype=torch.int32, device="cuda") for v in (block_expert, block_row0, block_rows)]
    got = ext.wq_gemv_batched(x, q, s, *plan, 0)
    assert got.shape == (rows, n)
    for e, r0, length in zip(block_expert[:8], block_row0[:8], lengths):
        want = oracle.gemv_float64(to_np(x[r0:r0 + length]), codes[e], stacks[e][1])
        assert rel_l2(to_np(got[r0:r0 + length]), want) <= 1e-2
        for r in range(r0, r0 + length):
            assert torch.equal(got[r], ext.wq_gemv(x[r:r + 1], q[e], s[e], 0)[0])
    assert not got[sum(lengths):].any()
    assert ext.wq_gemv_batched_max_rows() == 8


def test_unusual_group_size_takes_the_fallback_kernel(ext):
    gen = torch.Generator().manual_seed(1)
    experts, n, k, gs = 3, 40, 192, 64
    w = (torch.randn(experts, n, k, generator=gen) * 0.02).to(torch.bfloat16)
    stacks = [oracle.canonical_weight(to_np(w[e]), 8, gs) for e in range(experts)]
    q = torch.from_numpy(np.stack([c for c, _ in stacks])).cuda()
    s = torch.from_numpy(np.stack([sc for _, sc in stacks])).cuda()
    x = torch.randn(5, k, generator=gen).cuda()
    plan = [torch.tensor(v, dtype=torch.int32, device="cuda") for v in ([2, 0], [0, 3], [3, 2])]
    got = ext.wq_gemv_batched(x, q, s, *plan, 0)
    want = np.concatenate([oracle.gemv_float64(to_np(x[:3]), *stacks[2]), oracle.gemv_float64(to_np(x[3:]), *stacks[0])])
    assert rel_l2(to_np(got), want) <= 1e-5


@pytest.mark.parametrize("bits", ["int8", "int4"])
@pytest.mark.parametrize("tokens", [1, 2, 8])
def test_kernel_block_agrees_with_real_mode_and_the_oracle(bits, tokens):
    dense, quant, real, cfg = kernel_block(bits)
    torch.manual_seed(0)
    hidden = torch.randn(tokens, cfg.hidden_size, device="cuda", dtype=torch.bfloat16)
    index, weights = routing(tokens, cfg.num_local_experts, cfg.num_experts_per_tok, seed=5)
    index, weights = index.cuda(), weights.cuda()
    with torch.no_grad():
        got, want_real, want_dense = quant(hidden, index, weights), real(hidden, index, weights), dense(hidden, index, weights)
    want = oracle.moe_experts_real(to_np(hidden), to_np(index), to_np(weights), to_np(quant.qgate_up),
                                   to_np(quant.sgate_up), to_np(quant.qdown), to_np(quant.sdown))
    assert rel_l2(to_np(got), want) <= 1e-2            # bf16 outputs, summed in an order atomics choose
    assert rel_l2(to_np(got), to_np(want_real)) <= 1e-2
    assert (got.float() - want_dense.float()).abs().max() < want_dense.float().abs().max() * (0.1 if bits == "int8" else 0.5)


def test_short_rows_fall_back_and_stay_within_tolerance():
    """hidden 256 / intermediate 128 (the reference's test block): two groups and one group per
    row, below what the matrix-core kernel takes."""
    dense, quant, real, cfg = kernel_block(hidden=256, inter=128)
    hidden = torch.randn(3, cfg.hidden_size, device="cuda", dtype=torch.bfloat16)
    index, weights = routing(3, cfg.num_local_experts, cfg.num_experts_per_tok, seed=7)
    with torch.no_grad():
        got, want = quant(hidden, index.cuda(), weights.cuda()), real(hidden, index.cuda(), weights.cuda())
    assert rel_l2(to_np(got), to_np(want)) <= 1e-2


def test_wide_batches_take_the_per_expert_path():
    _, quant, real, cfg = kernel_block(experts=2, top_k=2)
    tokens = 64
    assert tokens > quant._batched_max_rows
    hidden = torch.randn(tokens, cfg.hidden_size, device="cuda", dtype=torch.bfloat16)
    index, weights = routing(tokens, cfg.num_local_experts, cfg.num_experts_per_tok)
    with torch.no_grad():
        out = quant(hidden, index.cuda(), weights.cuda())
        want = real(hidden, index.cuda(), weights.cuda())
    assert out.shape == hidden.shape and rel_l2(to_np(out), to_np(want)) <= 2e-2


def test_the_expert_block_replays_from_a_graph():
    _, quant, _, cfg = kernel_block()
    hidden = torch.randn(1, cfg.hidden_size, device="cuda", dtype=torch.bfloat16)
    index, weights = routing(1, cfg.num_local_experts, cfg.num_experts_per_tok)
    index, weights = index.cuda(), weights.cuda()
    with torch.no_grad():
        eager = quant(hidden, index, weights)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                quant(hidden, index, weights)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            captured = quant(hidden, index, weights)
        for _ in range(3):  # replays, each checked, with other work in between
            captured.zero_()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(captured, eager)
            quant(torch.randn_like(hidden), index, weights)
        index.copy_(torch.roll(index, 1, dims=1))  # the plan is rebuilt on the device inside the graph
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(captured, quant(hidden, index, weights))


def test_a_small_mixtral_in_kernel_mode_and_through_a_packed_file(tmp_path):
    from transformers import MixtralForCausalLM

    from llmquant.packing import load_packed_model, save_packed_model
    from llmquant.quantizers import KernelQuantExperts

    recipe = QuantConfig(attn_weight="int8", mlp_weight="int4", head_weight="int8")
    real = oneshot(mixtral_model().cuda(), recipe.to_modifier(mode="real"))
    kernel = oneshot(mixtral_model().cuda(), recipe.to_modifier(mode="kernel"))
    block = kernel.model.layers[0].mlp.experts
    assert isinstance(block, KernelQuantExperts) and block.gate_up_data.dtype == torch.uint8
    ids = torch.randint(0, 1000, (1, 6), generator=torch.Generator().manual_seed(3)).cuda()
    with torch.no_grad():
        want, got = real(ids).logits.float(), kernel(ids).logits.float()
    assert rel_l2(to_np(got), to_np(want)) <= 3e-2
    path = save_packed_model(kernel, tmp_path / "moe.llmq", "local-mixtral")
    loaded = load_packed_model(path, device="cuda", config=kernel.config)
    again = loaded.model.layers[0].mlp.experts
    assert isinstance(again, KernelQuantExperts)
    assert torch.equal(again.gate_up_data, block.gate_up_data) and torch.equal(again.sdown, block.sdown)
    with torch.no_grad():
        assert torch.equal(loaded(ids).logits, kernel(ids).logits)


@pytest.mark.parametrize("tokens,top_k,experts,limit", [(1, 8, 64, 8), (8, 8, 64, 8), (3, 2, 8, 8), (5, 4, 60, 3),
                                                         (64, 8, 64, 8), (1, 1, 1, 8), (700, 8, 128, 8), (9, 2, 1000, 4)])
def test_route_plan_kernel_matches_the_pytorch_form(tokens, top_k, experts, limit):
    """One launch against the argsort / scatter_add / cumsum form (itself pinned to the oracle on the CPU):
    the same order and the same blocks, for one token, many tokens, experts nobody picked, runs longer than
    the limit and a limit that does not divide them."""
    from llmquant.hip import load_extension
    from llmquant.quantizers import route_plan

    ext = load_extension()
    gen = torch.Generator().manual_seed(tokens * 131 + experts)
    index = torch.stack([torch.randperm(experts, generator=gen)[:top_k] for _ in range(tokens)]).cuda()
    assert ext.route_plan_supported(index.numel(), experts)
    for idx in (index, index.to(torch.int32)):
        order, be, r0, rows = ext.route_plan(idx, experts, limit)
        want_order, (want_be, want_r0, want_rows) = route_plan(index, experts, limit)
        assert order.dtype == torch.int64 and be.dtype == torch.int32
        assert torch.equal(order, want_order)
        assert torch.equal(be, want_be) and torch.equal(r0, want_r0) and torch.equal(rows, want_rows)
    # a skewed routing: every token picks the same experts, so their runs exceed the limit
    same = torch.arange(top_k).repeat(tokens, 1).cuda() % experts
    order, be, r0, rows = ext.route_plan(same, experts, limit)
    want_order, want = route_plan(same, experts, limit)
    assert torch.equal(order, want_order)
    assert all(torch.equal(a, b) for a, b in zip((be, r0, rows), want))


def test_route_plan_kernel_limits():
    from llmquant.hip import load_extension

    ext = load_extension()
    assert not ext.route_plan_supported(8193, 64)
    assert not ext.route_plan_supported(8, 1025)
    with pytest.raises(RuntimeError, match="does not take"):
        ext.route_plan(torch.zeros(8193, dtype=torch.int64, device="cuda"), 64, 8)
    with pytest.raises(RuntimeError, match="limit must be positive"):
        ext.route_plan(torch.zeros(8, dtype=torch.int64, device="cuda"), 64, 0)
    order, be, r0, rows = ext.route_plan(torch.zeros(0, dtype=torch.int64, device="cuda"), 4, 8)
    assert order.numel() == 0 and be.tolist() == [0, 1, 2, 3] and rows.tolist() == [0, 0, 0, 0]


@pytest.mark.parametrize("bits", ["int8", "int4"])
@pytest.mark.parametrize("tokens", [1, 3, 8])
def test_fused_forward_pieces_equal_the_operation_by_operation_form(ext, bits, tokens):
    """gate|up with act(gate) * up in its store, the one-token form that skips the row gather, and the
    weighted sum per token, each against the PyTorch steps of KernelQuantExperts.forward."""
    _, quant, _, cfg = kernel_block(bits)
    top_k = cfg.num_experts_per_tok
    torch.manual_seed(10 + tokens)
    hidden = torch.randn(tokens, cfg.hidden_size, device="cuda", dtype=torch.bfloat16)
    index, weights = routing(tokens, cfg.num_local_experts, top_k, seed=tokens)
    index, weights = index.cuda(), weights.to(torch.bfloat16).cuda()
    assert quant._fusable(hidden, index, weights)
    with torch.no_grad():
        order, plan = quant._plan(index)
        rows = hidden[order // top_k]
        plain = quant._batched(rows, quant.gate_up_data, quant.sgate_up, plan, quant.hidden_dim, quant._gate_up_padded)
        gate, up = plain.chunk(2, dim=-1)
        want_act = torch.nn.functional.silu(gate) * up
        act = ext.wq_gemv_batched_fused(rows, False, rows.shape[0], quant.gate_up_data, quant.sgate_up, *plan, True)
        assert torch.equal(act, want_act)
        if tokens == 1:
            again = ext.wq_gemv_batched_fused(hidden, True, rows.shape[0], quant.gate_up_data, quant.sgate_up, *plan, True)
            assert torch.equal(again, want_act)
        out = ext.wq_gemv_batched_fused(act, False, rows.shape[0], quant.down_data, quant.sdown, *plan, False)
        assert torch.equal(out, quant._batched(act, quant.down_data, quant.sdown, plan, quant.intermediate_dim,
                                               quant._down_padded))
        # index_add_ on a bf16 tensor rounds after every addition, in no fixed order; the kernel takes the
        # order of the sorted rows
        final = torch.zeros_like(hidden)
        flat_w = weights.reshape(-1)
        for i, src in enumerate(order.tolist()):
            final[src // top_k] = final[src // top_k] + out[i] * flat_w[src]
        got = ext.moe_combine(out, order, weights, tokens)
        assert torch.equal(got, final)
        assert torch.equal(quant._forward_fused(hidden, index, weights), final)
        loose = quant._forward_unfused(hidden, index, weights)
        assert rel_l2(to_np(got), to_np(loose)) <= 1e-2


def test_experts_that_are_not_silu_keep_the_unfused_forward(ext):
    _, quant, _, cfg = kernel_block("int8")
    assert quant._probe_silu()
    quant.act_fn = torch.nn.GELU()
    quant._act_is_silu = quant._probe_silu()
    hidden = torch.randn(2, cfg.hidden_size, device="cuda", dtype=torch.bfloat16)
    index, weights = routing(2, cfg.num_local_experts, cfg.num_experts_per_tok, seed=3)
    index, weights = index.cuda(), weights.to(torch.bfloat16).cuda()
    assert not quant._fusable(hidden, index, weights)
    assert torch.isfinite(quant(hidden, index, weights)).all()
