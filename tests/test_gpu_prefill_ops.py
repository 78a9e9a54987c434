"""The one-launch RMSNorm, RoPE and SiLU * up of a prompt pass against the transformers modules and
functions they replace (LlamaRMSNorm.forward, apply_rotary_pos_emb, act_fn(gate) * up): the same
rounding points, so equal to the bit except where the fp32 mean of squares is summed in another order
(RMSNorm: at most one unit in the last place of a few elements)."""

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ext():
    from llmquant.hip import load_extension

    return load_extension()


def ulps(a, b):
    """Elementwise distance in units of the last place of a 16-bit tensor."""
    ia = a.view(torch.int16).to(torch.int32)
    ib = b.view(torch.int16).to(torch.int32)
    ia = torch.where(ia < 0, -(ia & 0x7fff), ia)
    ib = torch.where(ib < 0, -(ib & 0x7fff), ib)
    return (ia - ib).abs()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("rows,hidden", [(1, 2048), (512, 2048), (7, 4096), (3, 136), (64, 8)])
def test_rmsnorm_matches_llama_rmsnorm(ext, dtype, rows, hidden):
    from transformers.models.llama.modeling_llama import LlamaRMSNorm

    torch.manual_seed(rows + hidden)
    norm = LlamaRMSNorm(hidden, eps=1e-5).to("cuda", dtype)
    with torch.no_grad():
        norm.weight.copy_(torch.randn(hidden) * 0.5 + 1.0)
    x = (torch.randn(rows, hidden, device="cuda") * 3.0).to(dtype)
    with torch.no_grad():
        want = norm(x)
    got = ext.rmsnorm(x, norm.weight, 1e-5)
    assert got.shape == want.shape and got.dtype == dtype
    if dtype == torch.float32:
        assert torch.allclose(got, want, rtol=2e-6, atol=0)
    else:
        d = ulps(got, want)
        assert int(d.max()) <= 1 and float((d > 0).float().mean()) < 0.02


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_add_rmsnorm_is_the_add_then_the_norm(ext, dtype):
    torch.manual_seed(4)
    x = (torch.randn(33, 1024, device="cuda") * 2.0).to(dtype)
    delta = torch.randn(33, 1024, device="cuda").to(dtype)
    w = (torch.randn(1024, device="cuda") * 0.3 + 1.0).to(dtype)
    total, normed = ext.add_rmsnorm(x, delta, w, 1e-5)
    assert torch.equal(total, x + delta)
    assert torch.equal(normed, ext.rmsnorm(x + delta, w, 1e-5))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("tokens,q_heads,kv_heads,head_dim", [(512, 32, 8, 64), (1, 32, 8, 64), (5, 8, 8, 128), (3, 4, 1, 16)])
def test_rope_matches_apply_rotary_pos_emb(ext, dtype, tokens, q_heads, kv_heads, head_dim):
    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb

    torch.manual_seed(tokens)
    q = torch.randn(tokens, q_heads * head_dim, device="cuda").to(dtype)
    k = torch.randn(tokens, kv_heads * head_dim, device="cuda").to(dtype)
    freqs = torch.rand(tokens, head_dim // 2, device="cuda") * 6.28
    emb = torch.cat((freqs, freqs), dim=-1)
    cos, sin = emb.cos().to(dtype), emb.sin().to(dtype)
    # transformers' layout: [batch, heads, tokens, D] with cos / sin [batch, tokens, D]
    q4 = q.view(1, tokens, q_heads, head_dim).transpose(1, 2)
    k4 = k.view(1, tokens, kv_heads, head_dim).transpose(1, 2)
    want_q, want_k = apply_rotary_pos_emb(q4, k4, cos[None], sin[None])
    got_q, got_k = ext.rope_qk(q, k, cos, sin, q_heads, kv_heads)
    assert got_q.shape == (tokens, q_heads, head_dim) and got_k.shape == (tokens, kv_heads, head_dim)
    assert torch.equal(got_q, want_q[0].transpose(0, 1)) and torch.equal(got_k, want_k[0].transpose(0, 1))


def test_rope_takes_strided_rows(ext):
    """q and k as column slices of one fused projection output."""
    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb

    torch.manual_seed(0)
    tokens, hq, hkv, d = 9, 4, 2, 64
    qkv = torch.randn(tokens, (hq + 2 * hkv) * d, device="cuda").to(torch.bfloat16)
    q, k = qkv[:, : hq * d], qkv[:, hq * d: (hq + hkv) * d]
    freqs = torch.rand(tokens, d // 2, device="cuda")
    emb = torch.cat((freqs, freqs), dim=-1)
    cos, sin = emb.cos().to(torch.bfloat16), emb.sin().to(torch.bfloat16)
    want_q, want_k = apply_rotary_pos_emb(q.reshape(1, tokens, hq, d).transpose(1, 2),
                                          k.reshape(1, tokens, hkv, d).transpose(1, 2), cos[None], sin[None])
    got_q, got_k = ext.rope_qk(q, k, cos, sin, hq, hkv)
    assert torch.equal(got_q, want_q[0].transpose(0, 1)) and torch.equal(got_k, want_k[0].transpose(0, 1))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(512, 8192), (1, 8), (3, 5, 64)])
def test_silu_mul_matches_the_mlp(ext, dtype, shape):
    from transformers.activations import ACT2FN

    torch.manual_seed(1)
    gate = (torch.randn(*shape, device="cuda") * 4.0).to(dtype)
    up = torch.randn(*shape, device="cuda").to(dtype)
    want = ACT2FN["silu"](gate) * up
    got = ext.silu_mul(gate, up)
    if dtype == torch.float32:
        assert torch.allclose(got, want, rtol=1e-6, atol=1e-7)
    else:
        d = ulps(got, want)  # (the exponential is evaluated by different routines)
        assert int(d.max()) <= 1 and float((d > 0).float().mean()) < 0.01


def test_silu_mul_takes_the_two_halves_of_one_projection(ext):
    from transformers.activations import ACT2FN

    torch.manual_seed(2)
    both = (torch.randn(37, 2 * 1024, device="cuda") * 3.0).to(torch.bfloat16)
    gate, up = both[:, :1024], both[:, 1024:]
    got = ext.silu_mul(gate, up)
    assert got.is_contiguous() and torch.equal(got, ext.silu_mul(gate.contiguous(), up.contiguous()))
    d = ulps(got, ACT2FN["silu"](gate) * up)
    assert int(d.max()) <= 1


def test_prompt_pass_with_one_projection_per_group_matches_the_module_walk():
    """LlamaFusedRuntime projects q|k|v and gate|up through the concatenated weights in a prompt pass;
    LlamaKernelRuntime calls the five modules: the same first token, and logits that agree to the
    rounding of two bf16 matmuls with different tilings."""
    from transformers import LlamaConfig, LlamaForCausalLM

    from llmquant import QuantConfig, oneshot
    from llmquant.runtime.llama_decode import LlamaKernelRuntime
    from llmquant.runtime.llama_fused import LlamaFusedRuntime

    torch.manual_seed(0)
    cfg = LlamaConfig(hidden_size=512, intermediate_size=1024, num_hidden_layers=2, num_attention_heads=8,
                      num_key_value_heads=2, head_dim=64, vocab_size=512, tie_word_embeddings=False,
                      max_position_embeddings=256)
    model = LlamaForCausalLM(cfg).to(torch.bfloat16).cuda().eval()
    oneshot(model, QuantConfig(attn_weight="int8", mlp_weight="int4", head_weight="int8", kv_cache="int8").to_modifier("kernel"))
    for tokens in (3, 40, 100):  # the GEMV's, the fused GEMM's and the dense branch's row counts
        ids = torch.randint(0, 512, (1, tokens), device="cuda")
        plain, fused = LlamaKernelRuntime(model, 128), LlamaFusedRuntime(model, 128)
        with torch.no_grad():
            plain.cache.set_position(0); plain.cache.length.fill_(tokens)
            a = plain._forward(ids[0], plain.cos_table[:tokens], plain.sin_table[:tokens], decode=False).float()
            fused.cache.set_position(0); fused.cache.length.fill_(tokens)
            b = fused._forward(ids[0], fused.cos_table[:tokens], fused.sin_table[:tokens], decode=False).float()
        assert float((a - b).norm() / a.norm()) < 3e-2
        assert torch.equal(plain.cache.k_codes[0, :, :tokens], fused.cache.k_codes[0, :, :tokens])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("tokens,q_heads,kv_heads,head_dim,start",
                         [(512, 32, 8, 64, 0), (5, 8, 8, 128, 3), (1, 4, 1, 64, 9), (37, 6, 2, 128, 0)])
def test_rope_and_append_in_one_launch_equal_the_two_launches(ext, dtype, bits, tokens, q_heads, kv_heads, head_dim, start):
    """llmq_rope_kv_append against llmq_rope_qk followed by llmq_kv_append (each tested on its own
    against transformers and the oracle): the same rotated query, codes, scales and dequantized K/V,
    to the bit, with q | k | v as column blocks of one projection output and a non-zero start position."""
    from llmquant.runtime.kv_cache import KernelQuantCache

    torch.manual_seed(tokens * 7 + head_dim + bits)
    qkv = (torch.randn(tokens, (q_heads + 2 * kv_heads) * head_dim, device="cuda") * 2.0).to(dtype)
    q_width, kv_width = q_heads * head_dim, kv_heads * head_dim
    q, k, v = qkv[:, :q_width], qkv[:, q_width:q_width + kv_width], qkv[:, q_width + kv_width:]
    freqs = torch.rand(tokens, head_dim // 2, device="cuda") * 6.28
    emb = torch.cat((freqs, freqs), dim=-1)
    cos, sin = emb.cos().to(dtype), emb.sin().to(dtype)
    max_len = start + tokens + 2
    two, one = (KernelQuantCache(1, kv_heads, head_dim, max_len, bits, q_heads=q_heads) for _ in range(2))
    two.set_position(start)
    one.set_position(start)

    want_q, rotated_k = ext.rope_qk(q, k, cos, sin, q_heads, kv_heads)
    want_k_dq, want_v_dq = two.append(0, rotated_k.transpose(0, 1),
                                      v.contiguous().view(tokens, kv_heads, head_dim).transpose(0, 1),
                                      return_dequantized=True)
    got_q, got_k_dq, got_v_dq = ext.rope_kv_append(q, k, v, cos, sin, one.k_codes[0], one.v_codes[0], one.k_scale[0],
                                                   one.v_scale[0], one.position, q_heads, True)
    assert got_q.shape == (tokens, q_heads, head_dim) and got_k_dq.shape == (kv_heads, tokens, head_dim)
    assert torch.equal(got_q, want_q)
    assert torch.equal(got_k_dq, want_k_dq) and torch.equal(got_v_dq, want_v_dq)
    assert torch.equal(one.k_codes, two.k_codes) and torch.equal(one.v_codes, two.v_codes)
    assert torch.equal(one.k_scale, two.k_scale) and torch.equal(one.v_scale, two.v_scale)
    assert float(one.k_scale[0, :, start:start + tokens].min()) > 0.0   # ... and something was written
    # without the dequantized copies: the same cache contents
    bare = KernelQuantCache(1, kv_heads, head_dim, max_len, bits, q_heads=q_heads)
    bare.set_position(start)
    _, none_k, none_v = ext.rope_kv_append(q, k, v, cos, sin, bare.k_codes[0], bare.v_codes[0], bare.k_scale[0],
                                           bare.v_scale[0], bare.position, q_heads, False)
    assert none_k.numel() == 0 and none_v.numel() == 0
    assert torch.equal(bare.k_codes, two.k_codes) and torch.equal(bare.v_scale, two.v_scale)


def test_rope_and_append_argument_checks(ext):
    from llmquant.runtime.kv_cache import KernelQuantCache

    cache = KernelQuantCache(1, 2, 64, 16, 8, q_heads=4)
    q = torch.randn(3, 4 * 64, device="cuda").to(torch.bfloat16)
    k = torch.randn(3, 2 * 64, device="cuda").to(torch.bfloat16)
    cos = torch.ones(3, 64, device="cuda", dtype=torch.bfloat16)
    args = (cache.k_codes[0], cache.v_codes[0], cache.k_scale[0], cache.v_scale[0], cache.position)
    with pytest.raises(RuntimeError, match="columns"):
        ext.rope_kv_append(q, k, k, cos, cos, *args, 3, True)
    with pytest.raises(RuntimeError, match="k and v must be"):
        ext.rope_kv_append(q, k[:2], k, cos, cos, *args, 4, True)
    with pytest.raises(RuntimeError, match="cos and sin"):
        ext.rope_kv_append(q, k, k, cos[:, :32].contiguous(), cos[:, :32].contiguous(), *args, 4, True)
    with pytest.raises(RuntimeError, match="share a dtype"):
        ext.rope_kv_append(q, k, k.float(), cos, cos, *args, 4, True)
    small = KernelQuantCache(1, 2, 32, 16, 8, q_heads=4)   # head_dim 32: the two-launch path's case
    with pytest.raises(RuntimeError, match="head_dim must be 64 or 128"):
        ext.rope_kv_append(q[:, :128].contiguous(), k[:, :64].contiguous(), k[:, :64].contiguous(),
                           cos[:, :32].contiguous(), cos[:, :32].contiguous(), small.k_codes[0], small.v_codes[0],
                           small.k_scale[0], small.v_scale[0], small.position, 4, True)
    out = ext.rope_kv_append(q[:0], k[:0], k[:0], cos[:0], cos[:0], *args, 4, True)
    assert out[0].shape == (0, 4, 64)


def test_argument_checks(ext):
    x = torch.randn(4, 64, device="cuda").to(torch.bfloat16)
    w = torch.ones(64, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="multiple of 8"):
        ext.rmsnorm(x[:, :60].contiguous(), w[:60].contiguous(), 1e-5)
    with pytest.raises(RuntimeError, match="weight must be"):
        ext.rmsnorm(x, w[:32].contiguous(), 1e-5)
    with pytest.raises(RuntimeError, match="must match"):
        ext.silu_mul(x, x[:2])
    with pytest.raises(RuntimeError, match="widths do not match"):
        ext.rope_qk(x, x, x[:, :16].contiguous(), x[:, :16].contiguous(), 2, 4)
    assert ext.rmsnorm(x[:0], w, 1e-5).shape == (0, 64)
