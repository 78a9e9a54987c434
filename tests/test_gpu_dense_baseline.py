"""The 16-bit baseline through the fused decode step: llmq_dense_gemv_fused (the decode-step GEMV over an
unquantized weight), the split attention launch over an unquantized cache (bits 16), and
LlamaDenseFusedRuntime, which runs a plain bf16 model through the same five launches per layer as the
quantized one so that the two are timed under one runtime (llmquant/eval/verify.py:44-47).

Anchors: numpy in float64 with the rounding points of transformers' decoder layer (oracle.llama_rmsnorm,
llama_gated_act, llama_residual_add), the oracle's grouped-query attention, and the HF model itself."""

import numpy as np
import pytest
import torch

import llmq_oracle as oracle
from conftest import rel_l2, to_np

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ext():
    from llmquant.hip import load_extension

    return load_extension()


def dense_case(n, k, dtype, seed):
    torch.manual_seed(seed)
    w = (torch.randn(n, k) * 0.02).to(dtype)
    x = (torch.randn(1, k) * 2).to(dtype)
    return w, x


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("n,k", [(3072, 2048), (2048, 8192), (4096, 14336), (1000, 4096), (37, 520), (128256, 2048)])
def test_dense_gemv_against_float64(ext, n, k, dtype):
    """Plain, with the RMSNorm prologue, and with the residual epilogue: every K-dependent form of the kernel
    (four, two and one row per wave step; rows that are not a whole number of wave loads; ragged N)."""
    tag = "bf16" if dtype == torch.bfloat16 else "f16"
    w, x = dense_case(n, k, dtype, seed=n + k)
    wf = to_np(w).astype(np.float64)
    got = ext.dense_gemv_fused(x.cuda(), w.cuda())
    assert got.shape == (1, n) and got.dtype == dtype
    assert rel_l2(to_np(got), to_np(x).astype(np.float64) @ wf.T) <= 2.5e-3
    norm = (1 + 0.1 * torch.randn(k)).to(dtype)
    res = torch.randn(1, n).to(dtype)
    got = ext.dense_gemv_fused(x.cuda(), w.cuda(), 1, norm.cuda(), 1e-5, res.cuda())
    staged = oracle.llama_rmsnorm(to_np(x), to_np(norm), 1e-5, tag).astype(np.float64)
    branch = oracle.round_to((staged @ wf.T).astype(np.float32), tag)
    want = oracle.llama_residual_add(to_np(res), branch, tag)
    assert rel_l2(to_np(got), want) <= 1e-2
    assert (to_np(got) == want).mean() > 0.97


@pytest.mark.parametrize("inter,k", [(8192, 2048), (14336, 4096), (100, 1024), (8, 16384)])
def test_dense_gate_up_store_against_float64(ext, inter, k):
    """pair_half: the gate|up weight with act(gate) * up stored, against LlamaMLP's elementwise step in numpy."""
    w, x = dense_case(2 * inter, k, torch.bfloat16, seed=inter)
    norm = (1 + 0.1 * torch.randn(k)).to(torch.bfloat16)
    got = ext.dense_gemv_fused(x.cuda(), w.cuda(), 1, norm.cuda(), 1e-5, None, inter)
    staged = oracle.llama_rmsnorm(to_np(x), to_np(norm), 1e-5, "bf16").astype(np.float64)
    both = oracle.round_to((staged @ to_np(w).astype(np.float64).T).astype(np.float32), "bf16")
    want = oracle.llama_gated_act(both[:, :inter], both[:, inter:], "bf16")
    assert got.shape == (1, inter)
    assert rel_l2(to_np(got), want) <= 1e-2
    assert (to_np(got) == want).mean() > 0.97


def test_dense_gemv_argument_checks(ext):
    w, x = dense_case(64, 256, torch.bfloat16, seed=1)
    with pytest.raises(RuntimeError, match="float16 or bfloat16"):
        ext.dense_gemv_fused(x.float().cuda(), w.float().cuda())
    with pytest.raises(RuntimeError, match="of the weight's dtype"):
        ext.dense_gemv_fused(x.cuda()[:, :128].contiguous(), w.cuda())
    with pytest.raises(RuntimeError, match="RMSNorm prologue needs"):
        ext.dense_gemv_fused(x.cuda(), w.cuda(), 1)
    with pytest.raises(RuntimeError, match="pair_half"):
        ext.dense_gemv_fused(x.cuda(), w.cuda(), 0, None, 0.0, None, 30)
    assert ext.dense_gemv_fused(x.cuda(), w.cuda()[:0]).shape == (1, 0)


def rope_reference(x, cos, sin):
    half = x.shape[-1] // 2
    rot = torch.cat((-x[..., half:], x[..., :half]), dim=-1)
    return (x * cos) + (rot * sin)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("q_heads,kv_heads,d", [(32, 8, 64), (8, 2, 128)])
@pytest.mark.parametrize("pos,splits", [(0, 8), (5, 2), (63, 8), (700, 8), (2047, 3)])
def test_split_attention_over_an_unquantized_cache(ext, q_heads, kv_heads, d, pos, splits, dtype):
    """bits 16: the cache holds the model dtype's values. What the launch appends is the rotated key and the value
    bit for bit; the merged output is the oracle's attention over those values (rel-L2 <= 1e-2); the o_proj GEMV
    that merges while staging equals merge-then-GEMV."""
    tag = "bf16" if dtype == torch.bfloat16 else "f16"
    torch.manual_seed(pos + splits)
    t_max = 2048
    kc = torch.zeros(kv_heads, t_max, d, dtype=dtype, device="cuda")
    vc = torch.zeros(kv_heads, t_max, d, dtype=dtype, device="cuda")
    ks, vs = torch.ones(kv_heads, t_max, device="cuda"), torch.ones(kv_heads, t_max, device="cuda")
    past_k = torch.randn(kv_heads, pos, d).to(dtype)
    past_v = torch.randn(kv_heads, pos, d).to(dtype)
    kc[:, :pos], vc[:, :pos] = past_k.cuda(), past_v.cuda()
    kc[:, pos + 1:], vc[:, pos + 1:] = float("nan"), float("nan")   # read ahead of the position, must be dropped
    inv_freq = 1.0 / (500000.0 ** (torch.arange(0, d, 2).float() / d))
    emb = torch.cat((torch.outer(torch.arange(t_max).float(), inv_freq),) * 2, -1)
    cos_t, sin_t = emb.cos().to(dtype), emb.sin().to(dtype)
    qkv = torch.randn(1, (q_heads + 2 * kv_heads) * d).to(dtype)
    position = torch.tensor([pos], dtype=torch.int32, device="cuda")
    partials = torch.full((ext.kv_attend_partials_floats(q_heads, d, splits),), float("nan"), device="cuda")
    ext.kv_rope_append_attend_split(qkv.cuda(), cos_t.cuda(), sin_t.cuda(), kc, vc, ks, vs, partials, position,
                                    d ** -0.5, q_heads, splits)
    q = qkv[0, : q_heads * d].view(q_heads, d)
    k = qkv[0, q_heads * d: (q_heads + kv_heads) * d].view(kv_heads, d)
    v = qkv[0, (q_heads + kv_heads) * d:].view(kv_heads, d)
    q_r, k_r = rope_reference(q, cos_t[pos], sin_t[pos]), rope_reference(k, cos_t[pos], sin_t[pos])
    assert torch.equal(kc[:, pos].cpu(), k_r) and torch.equal(vc[:, pos].cpu(), v)
    assert torch.equal(kc[:, :pos].cpu(), past_k)   # earlier rows untouched
    merged = ext.kv_attend_merge(partials, q_heads, d, splits, dtype)
    keys = np.concatenate([to_np(past_k), to_np(k_r)[:, None]], axis=1)
    values = np.concatenate([to_np(past_v), to_np(v)[:, None]], axis=1)
    want = oracle.gqa_decode_attention(to_np(q_r), keys, values, d ** -0.5, tag)
    assert torch.isfinite(merged.float()).all()
    assert rel_l2(to_np(merged).reshape(q_heads, d), want) <= 1e-2
    w, _ = dense_case(256, q_heads * d, dtype, seed=3)
    res = torch.randn(1, 256).to(dtype).cuda()
    got = ext.dense_gemv_fused(partials, w.cuda(), 3, None, 0.0, res, 0, splits, d)
    assert torch.equal(got, ext.dense_gemv_fused(merged, w.cuda(), 0, None, 0.0, res))


def build_bf16(hidden, inter, layers, heads, kv_heads, vocab, seed=0, head_dim=64):
    from test_gpu_decode import build_model

    return build_model(hidden, inter, layers, heads, kv_heads, vocab, seed=seed, head_dim=head_dim)


@pytest.mark.parametrize("shape,head_dim", [((512, 1024, 3, 8, 2, 4096), 64), ((512, 2048, 2, 4, 2, 4096), 128)])
def test_dense_fused_runtime_tracks_the_hf_model(shape, head_dim):
    """A plain bf16 model through LlamaDenseFusedRuntime against the same model under HF transformers, teacher-forced
    on HF's own greedy stream: logits within 5 % relative and every differing pick at an HF top-2 gap within twice
    the logit error there (two bf16 implementations of one model). Graph replay equals eager execution to the bit."""
    from test_gpu_decode import check_margin

    from llmquant.runtime import LlamaDenseFusedRuntime, graphed_generate, kernel_runtime

    model = build_bf16(*shape, seed=4, head_dim=head_dim)
    prompt, new = 70, 24
    ids = torch.randint(0, 4096, (1, prompt), generator=torch.Generator().manual_seed(1)).cuda()
    from transformers import DynamicCache

    cache = DynamicCache()
    with torch.no_grad():
        want = model(ids, past_key_values=cache, use_cache=True).logits[0, -1]
    rt = LlamaDenseFusedRuntime(model, prompt + new + 2)
    assert isinstance(kernel_runtime(model, prompt + new + 2, 16), LlamaDenseFusedRuntime)
    first = rt.prefill(ids)
    rows = [(first.item() == want.argmax().item(), 0.0, 0.0, 0.0)]
    tok = want.argmax().reshape(1)
    for i in range(new):
        with torch.no_grad():
            want = model(tok.reshape(1, 1), past_key_values=cache, use_cache=True).logits[0, -1].float()
        logits, nxt = rt.eager_step(tok, prompt + i)
        got = logits[0].float()
        top2 = want.topk(2).values
        rows.append((nxt.item() == want.argmax().item(), (top2[0] - top2[1]).item(),
                     (got - want).abs().max().item(), ((got - want).norm() / want.norm()).item()))
        tok = want.argmax().reshape(1)
    agree = check_margin(rows, 0.05)
    print(f"dense fused runtime vs HF, heads of {head_dim}: {agree}/{len(rows)} picks equal")
    assert agree >= 0.8 * len(rows)
    replay = graphed_generate(model, ids, new, kv_bits=16)
    eager = LlamaDenseFusedRuntime(model, prompt + new + 1).generate(ids, new, use_graph=False)
    assert torch.equal(replay, eager)
    model.__dict__.pop("_llmq_kept_runtimes", None)


def test_dense_fused_runtime_refuses_what_it_does_not_take():
    from test_gpu_decode import quantized_pair

    from llmquant.runtime import LlamaDenseFusedRuntime

    model = build_bf16(256, 512, 1, 4, 2, 1024)
    with pytest.raises(ValueError, match="kv_bits 16"):
        LlamaDenseFusedRuntime(model, 64, 8)
    _, kernel = quantized_pair(model)
    with pytest.raises(ValueError, match="plain 16-bit nn.Linear"):
        LlamaDenseFusedRuntime(kernel, 64)
    with pytest.raises(ValueError, match="bfloat16 or float16"):
        LlamaDenseFusedRuntime(model.float(), 64)
