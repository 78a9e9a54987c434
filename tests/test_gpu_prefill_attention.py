"""Causal grouped-query attention of a prompt (llmq_prefill_attention) against the oracle's float64
restatement (oracle.gqa_prompt_attention), and against torch's scaled_dot_product_attention, which is what the
reference's prompt pass runs on the K / V its FakeQuantCache returns (llmquant/quantizers/fake.py:39-55).

Floating point, so a tolerance: the kernel accumulates scores and the weighted sum in fp32 and rounds the
probabilities to the 16-bit type before they meet V, as the library's flash kernel does. Against float64 the
error of an output element is therefore a few units in the last place of the 16-bit type at the output's
magnitude: the tests ask for |got - want| <= 2^-7 |want| + 2^-8 (bf16) or 2^-10 |want| + 2^-11 (fp16) with
|v| <= ~4, and that the kernel is no further from float64 than 1.5 x the library's own distance plus one ulp."""

import math

import numpy as np
import pytest
import torch

import llmq_oracle as oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ext():
    from llmquant.hip import load_extension

    return load_extension()


def causal_gqa_float64(q, k, v, scale):
    """q [T, Hq, D]; k, v [Hkv, T, D] (16-bit tensors on the CPU) -> [T, Hq * D] in float64: the oracle's
    restatement of what the reference's prompt pass computes."""
    return torch.from_numpy(oracle.gqa_prompt_attention(q.float().numpy(), k.float().numpy(), v.float().numpy(), scale))


def make(tokens, q_heads, kv_heads, d, dtype, seed, spread=1.0):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(tokens, q_heads, d, generator=g) * spread).to(dtype)
    k = (torch.randn(kv_heads, tokens, d, generator=g) * spread).to(dtype)
    v = torch.randn(kv_heads, tokens, d, generator=g).to(dtype)
    return q, k, v


TOL = {torch.bfloat16: (2.0 ** -7, 2.0 ** -8), torch.float16: (2.0 ** -10, 2.0 ** -11)}


def check(ext, q, k, v, scale):
    want = causal_gqa_float64(q, k, v, scale)
    got = ext.prefill_attention(q.cuda(), k.cuda(), v.cuda(), scale)
    assert got.shape == want.shape and got.dtype == q.dtype
    got = got.double().cpu()
    assert torch.isfinite(got).all()
    rtol, atol = TOL[q.dtype]
    err = (got - want).abs()
    bound = rtol * want.abs() + atol
    worst = int(torch.argmax(err - bound))
    assert bool((err <= bound).all()), (float(err.flatten()[worst]), float(want.flatten()[worst]), worst)
    return got, want


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("tokens,q_heads,kv_heads,d", [
    (512, 32, 8, 64),     # Llama-3.2-1B's prompt in the benchmark
    (128, 8, 2, 128),     # Llama-3-8B's head shape
    (1, 4, 4, 64), (2, 4, 1, 64), (31, 4, 2, 128), (32, 2, 2, 64), (33, 6, 2, 64), (63, 2, 1, 128),
    (64, 3, 3, 64), (65, 4, 2, 64), (97, 8, 8, 128), (200, 4, 1, 64), (257, 2, 2, 128),
    # long walks: many blocks per wave, head counts that are no multiple of four
    (1023, 4, 1, 64), (1024, 8, 2, 64), (1100, 6, 2, 64), (1025, 5, 5, 128), (1300, 4, 4, 128), (2048, 8, 2, 64),
])
def test_matches_float64_causal_gqa(ext, dtype, tokens, q_heads, kv_heads, d):
    q, k, v = make(tokens, q_heads, kv_heads, d, dtype, seed=tokens * 7 + d)
    check(ext, q, k, v, 1.0 / math.sqrt(d))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_peaked_softmax_and_large_scores(ext, dtype):
    """Scores tens of units apart: the running maximum has to move, and old sums have to be scaled away."""
    q, k, v = make(160, 4, 2, 64, dtype, seed=3, spread=3.0)
    check(ext, q, k, v, 0.5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("tokens,q_heads,kv_heads,d", [(512, 32, 8, 64), (300, 8, 2, 128), (77, 4, 4, 64), (1536, 8, 2, 64)])
def test_no_further_from_float64_than_the_library(ext, dtype, tokens, q_heads, kv_heads, d):
    q, k, v = make(tokens, q_heads, kv_heads, d, dtype, seed=11)
    scale = 1.0 / math.sqrt(d)
    got, want = check(ext, q, k, v, scale)
    lib = torch.nn.functional.scaled_dot_product_attention(
        q.cuda().transpose(0, 1)[None], k.cuda()[None], v.cuda()[None], is_causal=True, scale=scale, enable_gqa=True)
    lib = lib[0].transpose(0, 1).reshape(tokens, -1).double().cpu()
    ours, theirs = (got - want).abs(), (lib - want).abs()
    ulp = TOL[dtype][1]
    assert float(ours.mean()) <= 1.5 * float(theirs.mean()) + 0.05 * ulp
    assert float(ours.max()) <= 1.5 * float(theirs.max()) + ulp


def test_first_query_sees_only_the_first_key_and_rows_do_not_depend_on_later_tokens(ext):
    """Closed forms: out[0] = v[:, 0]; and the output of query i is unchanged when the prompt grows."""
    q, k, v = make(150, 4, 2, 64, torch.bfloat16, seed=5)
    full = ext.prefill_attention(q.cuda(), k.cuda(), v.cuda(), 0.125)
    first = full[0].view(4, 64).cpu()
    assert torch.equal(first[0], v[0, 0]) and torch.equal(first[1], v[0, 0])
    assert torch.equal(first[2], v[1, 0]) and torch.equal(first[3], v[1, 0])
    for shorter in (1, 31, 64, 100):
        part = ext.prefill_attention(q[:shorter].cuda(), k[:, :shorter].contiguous().cuda(),
                                     v[:, :shorter].contiguous().cuda(), 0.125)
        assert torch.equal(part, full[:shorter])
    # the same on a long prompt
    q, k, v = make(1500, 4, 2, 64, torch.bfloat16, seed=6)
    full = ext.prefill_attention(q.cuda(), k.cuda(), v.cuda(), 0.125)
    part = ext.prefill_attention(q[:1111].cuda(), k[:, :1111].contiguous().cuda(), v[:, :1111].contiguous().cuda(), 0.125)
    assert torch.equal(part, full[:1111])


def test_equal_keys_give_the_running_mean_of_v(ext):
    """All keys equal: the softmax is uniform over the open keys and out[i] = mean(v[:i + 1])."""
    tokens, d = 96, 64
    g = torch.Generator().manual_seed(9)
    q = torch.randn(tokens, 2, d, generator=g).to(torch.float16)
    k = torch.randn(1, 1, d, generator=g).expand(1, tokens, d).contiguous().to(torch.float16)
    v = torch.randn(1, tokens, d, generator=g).to(torch.float16)
    got = ext.prefill_attention(q.cuda(), k.cuda(), v.cuda(), 0.3).double().cpu().view(tokens, 2, d)
    want = v[0].double().cumsum(0) / torch.arange(1, tokens + 1, dtype=torch.float64)[:, None]
    for h in range(2):
        assert torch.allclose(got[:, h], want, rtol=2.0 ** -9, atol=2.0 ** -9)


def test_empty_prompt_and_argument_checks(ext):
    q = torch.empty(0, 4, 64, dtype=torch.bfloat16, device="cuda")
    kv = torch.empty(2, 0, 64, dtype=torch.bfloat16, device="cuda")
    assert ext.prefill_attention(q, kv, kv, 1.0).shape == (0, 256)
    q, k, v = (t.cuda() for t in make(8, 4, 2, 64, torch.bfloat16, seed=1))
    with pytest.raises(RuntimeError, match="head_dim"):
        ext.prefill_attention(q[..., :32].contiguous(), k[..., :32].contiguous(), v[..., :32].contiguous(), 1.0)
    with pytest.raises(RuntimeError, match="multiple"):
        ext.prefill_attention(q[:, :3].contiguous(), k, v, 1.0)
    with pytest.raises(RuntimeError, match="float16 or bfloat16"):
        ext.prefill_attention(q.float(), k.float(), v.float(), 1.0)
    with pytest.raises(RuntimeError, match="positive"):
        ext.prefill_attention(q, k, v, -1.0)
    with pytest.raises(RuntimeError, match="k and v must be"):
        ext.prefill_attention(q, k[:, :4].contiguous(), v[:, :4].contiguous(), 1.0)


def test_through_the_c_abi(ext):
    """The same call through libllmq_hip.so with raw pointers."""
    from llmquant.hip.build import load_capi

    lib = load_capi()
    q, k, v = (t.cuda() for t in make(70, 4, 2, 64, torch.bfloat16, seed=2))
    out = torch.empty(70, 256, dtype=torch.bfloat16, device="cuda")
    torch.cuda.synchronize()
    rc = lib.llmq_prefill_attention(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), 70, 4, 2, 64, 0.125, 2, None)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(out, ext.prefill_attention(q, k, v, 0.125))
    assert lib.llmq_prefill_attention(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), 70, 4, 3, 64, 0.125, 2, None) != 0
    assert b"multiple" in lib.llmq_last_error()
