"""The fused decode-step kernels: against the CPU oracle, and against the operation-by-operation forms
they replace.

Each fused op must reproduce the PyTorch sequence of transformers' LlamaDecoderLayer with its
rounding points: RMSNorm -> Linear, SiLU(gate)*up -> Linear, head-padded input -> Linear,
Linear -> + residual, RoPE -> cache append -> attention, argmax.

The oracle tests (`*_against_the_oracle`) build the staged activation in numpy with the library's rounding
points (oracle.llama_rmsnorm / llama_gated_act / pad_activation / llama_residual_add, themselves pinned
against transformers' modules on the CPU) and hold the kernel's output to the float64 closed form of the
real-mode Linear (llmquant/quantizers/real.py:76-103) at the Llama-3.2-1B and Llama-3-8B layer shapes, int8
and int4: rel-L2 <= 1e-2 for bf16 outputs and <= 1e-3 for fp32 (the stated bars; measured ~2e-3 and ~1e-7).
The remaining tests compare with the unfused sequence over the same GEMV / cache kernels, where equality is
expected to the bit except where a reduction order differs (RMSNorm's variance).
"""

import numpy as np
import pytest
import torch

import llmq_oracle as oracle
from conftest import rel_l2, to_np

pytestmark = pytest.mark.gpu
GROUP = 128


@pytest.fixture(scope="module")
def ext():
    from llmquant.hip import load_extension

    return load_extension()


def weights(n, k, bits, out_group=0, head_dim=None, seed=0):
    torch.manual_seed(seed)
    w = (torch.randn(n, k) * 0.02).to(torch.bfloat16)
    canonical, scales = oracle.canonical_weight(to_np(w), bits, GROUP, head_dim, out_group or None)
    q = torch.from_numpy(oracle.pack_int4(canonical) if bits == 4 else canonical).cuda()
    return q, torch.from_numpy(scales).cuda()


def oracle_weights(n, k, bits, out_group=0, head_dim=None, seed=0):
    """(device codes, device scales, canonical codes, scales): the weight on both sides of a comparison."""
    torch.manual_seed(seed)
    w = (torch.randn(n, k) * 0.02).to(torch.bfloat16)
    canonical, scales = oracle.canonical_weight(to_np(w), bits, GROUP, head_dim, out_group or None)
    q = torch.from_numpy(oracle.pack_int4(canonical) if bits == 4 else canonical).cuda()
    return q, torch.from_numpy(scales).cuda(), canonical, scales


#: the projections a decode step runs behind an RMSNorm, (N, K, out_group): q|k|v with one scale row per head,
#: gate|up, lm_head -- of the Llama-3.2-1B and the Llama-3-8B architecture
NORM_THEN_LINEAR = {
    "1B q|k|v": (3072, 2048, 64), "1B gate|up": (16384, 2048, 0), "1B lm_head": (128256, 2048, 0),
    "8B q|k|v": (6144, 4096, 128), "8B gate|up": (28672, 4096, 0),
}


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("name", list(NORM_THEN_LINEAR))
def test_rmsnorm_prologue_against_the_oracle(ext, name, bits, dtype):
    """llmq_wq_gemv_fused with the RMSNorm prologue == real-mode Linear over LlamaRMSNorm's output, both in
    numpy: the norm with the library's rounding points, the Linear as the float64 closed form."""
    n, k, out_group = NORM_THEN_LINEAR[name]
    q, s, canonical, scales = oracle_weights(n, k, bits, out_group, seed=21)
    tag = "bf16" if dtype == torch.bfloat16 else "f32"
    torch.manual_seed(22)
    x = (torch.randn(1, k) * 3).to(dtype)
    norm = (1 + 0.1 * torch.randn(k)).to(dtype)
    got = ext.wq_gemv_fused(x.cuda(), q, s, out_group, 1, norm.cuda(), 1e-5, 0, None)
    assert got.shape == (1, n) and got.dtype == dtype
    staged = oracle.llama_rmsnorm(to_np(x), to_np(norm), 1e-5, tag)
    exact = oracle.gemv_float64(staged, canonical, scales, out_group or None)
    err = rel_l2(to_np(got), exact)
    assert err <= (1e-2 if tag == "bf16" else 1e-3)
    assert err <= (2.5e-3 if tag == "bf16" else 1e-5)   # measured: the output's own rounding and little else
    if tag == "bf16":
        want = oracle.round_to(exact.astype(np.float32), "bf16")
        assert (to_np(got) == want).mean() > 0.98


#: down_proj of the two architectures: (N, K)
GATED_THEN_LINEAR = {"1B down": (2048, 8192), "8B down": (4096, 14336)}


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("name", list(GATED_THEN_LINEAR))
def test_silu_mul_prologue_and_residual_against_the_oracle(ext, name, bits):
    """llmq_wq_gemv_fused with the SiLU(gate) * up prologue and the residual epilogue == LlamaMLP's elementwise
    step, the real-mode Linear and LlamaDecoderLayer's add, each with its bf16 rounding, in numpy."""
    n, k = GATED_THEN_LINEAR[name]
    q, s, canonical, scales = oracle_weights(n, k, bits, seed=23)
    torch.manual_seed(24)
    gate_up = (torch.randn(1, 2 * k) * 2).to(torch.bfloat16)
    res = torch.randn(1, n).to(torch.bfloat16)
    got = ext.wq_gemv_fused(gate_up.cuda(), q, s, 0, 2, None, 0.0, 0, res.cuda())
    act = oracle.llama_gated_act(to_np(gate_up)[:, :k], to_np(gate_up)[:, k:], "bf16")
    branch = oracle.gemv_float64(act, canonical, scales)
    want = oracle.llama_residual_add(to_np(res), oracle.round_to(branch.astype(np.float32), "bf16"), "bf16")
    assert rel_l2(to_np(got), want) <= 1e-2
    assert rel_l2(to_np(got), to_np(res).astype(np.float64) + branch) <= 3e-3   # (unrounded: the tolerance anchor)
    assert (to_np(got) == want).mean() > 0.98
    # and with nothing in front of it but the residual behind: the plain activation
    plain = ext.wq_gemv_fused(torch.from_numpy(act).to(torch.bfloat16).cuda(), q, s, 0, 0, None, 0.0, 0, res.cuda())
    assert rel_l2(to_np(plain), want) <= 1e-2 and (to_np(plain) == want).mean() > 0.98


@pytest.mark.parametrize("prologue", [0, 1], ids=["plain", "rmsnorm"])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("inter,k", [(8192, 2048), (14336, 4096)], ids=["1B gate|up", "8B gate|up"])
def test_gate_up_silu_against_the_oracle(ext, inter, k, bits, prologue):
    """llmq_wq_gemv_gate_up_silu (the gate|up GEMV that stores act(gate) * up) == [RMSNorm ->] the two real-mode
    Linears -> LlamaMLP's elementwise step, in numpy: gate and up rounded to bf16 as the Linears' outputs are,
    silu rounded, the product rounded."""
    q, s, canonical, scales = oracle_weights(2 * inter, k, bits, seed=25)
    torch.manual_seed(26)
    x = (torch.randn(1, k) * 2).to(torch.bfloat16)
    norm = (1 + 0.1 * torch.randn(k)).to(torch.bfloat16) if prologue else None
    got = ext.wq_gemv_gate_up_silu(x.cuda(), q, s, prologue, norm.cuda() if prologue else None, 1e-5)
    staged = oracle.llama_rmsnorm(to_np(x), to_np(norm), 1e-5, "bf16") if prologue else to_np(x)
    both = oracle.round_to(oracle.gemv_float64(staged, canonical, scales).astype(np.float32), "bf16")
    want = oracle.llama_gated_act(both[:, :inter], both[:, inter:], "bf16")
    assert got.shape == (1, inter)
    assert rel_l2(to_np(got), want) <= 1e-2
    assert (to_np(got) == want).mean() > 0.97


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("n,k,head_dim", [(2048, 2048, 64), (4096, 4096, 128)], ids=["1B o_proj", "8B o_proj"])
def test_head_padding_and_residual_against_the_oracle(ext, n, k, head_dim, bits):
    """o_proj in the decode step: the attention output's heads padded to groups while staging (heads of 64 in
    groups of 128; heads of 128 need none), the real-mode Linear, the residual add -- against numpy."""
    padded_heads = head_dim if head_dim < GROUP else None
    q, s, canonical, scales = oracle_weights(n, k, bits, head_dim=padded_heads, seed=27)
    torch.manual_seed(28)
    x = torch.randn(1, k).to(torch.bfloat16)
    res = torch.randn(1, n).to(torch.bfloat16)
    got = ext.wq_gemv_fused(x.cuda(), q, s, 0, 0, None, 0.0, padded_heads or 0, res.cuda())
    branch = oracle.gemv_float64(oracle.pad_activation(to_np(x), GROUP, padded_heads), canonical, scales)
    want = oracle.llama_residual_add(to_np(res), oracle.round_to(branch.astype(np.float32), "bf16"), "bf16")
    assert rel_l2(to_np(got), want) <= 1e-2
    assert (to_np(got) == want).mean() > 0.98


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("n,k", [(3072, 2048), (16384, 2048), (128256, 2048), (2048, 4096)])
def test_rmsnorm_prologue(ext, bits, n, k):
    q, s = weights(n, k, bits)
    torch.manual_seed(1)
    x = (torch.randn(1, k) * 3).to(torch.bfloat16).cuda()
    norm = torch.nn.Parameter((1 + 0.1 * torch.randn(k)).to(torch.bfloat16).cuda())
    eps = 1e-5
    got = ext.wq_gemv_fused(x, q, s, 0, 1, norm, eps, 0, None)
    xf = x.float()
    normed = norm * (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).to(torch.bfloat16)  # LlamaRMSNorm
    want = ext.wq_gemv(normed, q, s, 0)
    assert got.shape == (1, n)
    assert rel_l2(to_np(got), to_np(want)) <= 2e-3  # only the variance's summation order may differ
    assert (got == want).float().mean() > 0.98


@pytest.mark.parametrize("bits", [8, 4])
def test_silu_mul_prologue_and_residual(ext, bits):
    n, k = 2048, 8192
    q, s = weights(n, k, bits)
    torch.manual_seed(2)
    gate_up = (torch.randn(1, 2 * k) * 2).to(torch.bfloat16).cuda()
    res = torch.randn(1, n).to(torch.bfloat16).cuda()
    got = ext.wq_gemv_fused(gate_up, q, s, 0, 2, None, 0.0, 0, res)
    act = torch.nn.functional.silu(gate_up[:, :k]) * gate_up[:, k:]  # LlamaMLP, bf16 roundings included
    want = res + ext.wq_gemv(act, q, s, 0)
    assert torch.equal(got, want)


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("inter,k", [(8192, 2048), (14336, 4096), (264, 512), (2056, 9216)])
@pytest.mark.parametrize("prologue", [0, 1])
def test_gate_up_silu_epilogue(ext, bits, inter, k, prologue):
    """gate|up GEMV that stores act(gate) * up == the plain GEMV followed by LlamaMLP's elementwise step.
    (8192, 2048) / (14336, 4096): the whole-row int4 kernels; 264: two tiles past a multiple of 16 rows;
    (2056, 9216): rows of 72 groups, the multi-chunk K-split kernel."""
    q, s = weights(2 * inter, k, bits, seed=5)
    torch.manual_seed(6)
    x = (torch.randn(1, k) * 2).to(torch.bfloat16).cuda()
    norm = (1 + 0.1 * torch.randn(k)).to(torch.bfloat16).cuda() if prologue else None
    got = ext.wq_gemv_gate_up_silu(x, q, s, prologue, norm, 1e-5)
    plain = ext.wq_gemv_fused(x, q, s, 0, prologue, norm, 1e-5, 0, None)
    want = torch.nn.functional.silu(plain[:, :inter]) * plain[:, inter:]
    assert got.shape == (1, inter)
    assert torch.equal(got, want)


def test_gate_up_silu_argument_checks(ext):
    q, s = weights(48, 512, 8)
    x = torch.randn(1, 512).to(torch.bfloat16).cuda()
    with pytest.raises(RuntimeError, match="multiples of 8"):
        ext.wq_gemv_gate_up_silu(x, q[:40].contiguous(), s[:40].contiguous(), 0, None, 0.0)
    with pytest.raises(RuntimeError, match="no prologue or RMSNorm"):
        ext.wq_gemv_gate_up_silu(x, q, s, 2, None, 0.0)
    with pytest.raises(RuntimeError, match="RMSNorm prologue needs"):
        ext.wq_gemv_gate_up_silu(x, q, s, 1, None, 0.0)
    assert ext.wq_gemv_gate_up_silu(x, q, s, 0, None, 0.0).shape == (1, 24)


@pytest.mark.parametrize("bits", [8, 4])
def test_head_padding_and_residual(ext, bits):
    """o_proj: 32 heads of 64 in groups of 128 (pad_activation), one scale group per head."""
    from llmquant.core.scheme import QuantizationArgs
    from llmquant.quantizers import pad_activation

    n, k = 2048, 2048
    q, s = weights(n, k, bits, head_dim=64)
    assert q.shape[1] == 32
    torch.manual_seed(3)
    x = torch.randn(1, k).to(torch.bfloat16).cuda()
    res = torch.randn(1, n).to(torch.bfloat16).cuda()
    got = ext.wq_gemv_fused(x, q, s, 0, 0, None, 0.0, 64, res)
    padded = pad_activation(x, QuantizationArgs(bits, "group", group_size=128, head_dim=64))
    want = res + ext.wq_gemv(padded, q, s, 0)
    assert torch.equal(got, want)
    q16, s16 = q[:, :16].contiguous(), s[:, :16].contiguous()
    plain = ext.wq_gemv_fused(x, q16, s16, 0, 0, None, 0.0, 0, None)
    assert torch.equal(plain, ext.wq_gemv(x, q16, s16, 0))


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("heads,head_dim", [(8, 64), (16, 64), (64, 64), (80, 64), (32, 32), (16, 96), (40, 8)])
def test_head_padding_widths(ext, bits, heads, head_dim):
    """Heads narrower than a group, each padded to a group of its own: every workgroup size of the int8
    form that skips the padded half (8 / 16 / 64 heads of 64 or less), rows too long for it (80 heads:
    the multi-chunk kernel), heads wider than half a group (96: nothing can be skipped), tiny heads."""
    from llmquant.core.scheme import QuantizationArgs
    from llmquant.quantizers import pad_activation

    n, k = 272, heads * head_dim
    q, s = weights(n, k, bits, head_dim=head_dim, seed=11)
    assert q.shape[1] == heads
    torch.manual_seed(12)
    x = torch.randn(1, k).to(torch.bfloat16).cuda()
    res = torch.randn(1, n).to(torch.bfloat16).cuda()
    got = ext.wq_gemv_fused(x, q, s, 0, 0, None, 0.0, head_dim, res)
    padded = pad_activation(x, QuantizationArgs(bits, "group", group_size=128, head_dim=head_dim))
    assert torch.equal(got, res + ext.wq_gemv(padded, q, s, 0))
    # what the padded half of the weight holds must not matter: the activation there is zero
    noisy = q.clone()
    if bits == 8:
        noisy[:, :, head_dim:] = 77
    else:
        noisy[:, :, (head_dim + 1) // 2:] = 0x5A
    assert torch.equal(ext.wq_gemv_fused(x, noisy, s, 0, 0, None, 0.0, head_dim, res), got)


def test_fused_gemv_argument_checks(ext):
    q, s = weights(256, 512, 8)
    x = torch.randn(1, 512, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="RMSNorm prologue needs"):
        ext.wq_gemv_fused(x, q, s, 0, 1, None, 1e-5, 0, None)
    with pytest.raises(RuntimeError, match="x has"):
        ext.wq_gemv_fused(x, q, s, 0, 2, None, 0.0, 0, None)
    with pytest.raises(RuntimeError, match="residual must be"):
        ext.wq_gemv_fused(x, q, s, 0, 0, None, 0.0, 0, torch.zeros(1, 8, device="cuda", dtype=torch.bfloat16))
    q3, s3 = weights(64, 384, 8)  # 3 groups: not a multiple of 4
    with pytest.raises(RuntimeError, match="multiple of 4 groups"):
        ext.wq_gemv_fused(torch.randn(1, 384, device="cuda", dtype=torch.bfloat16), q3, s3, 0, 0, None, 0.0, 0, None)


def rope_reference(x, cos, sin):
    half = x.shape[-1] // 2
    rot = torch.cat((-x[..., half:], x[..., :half]), dim=-1)
    return (x * cos) + (rot * sin)


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("q_heads,kv_heads,d", [(32, 8, 64), (8, 8, 64), (8, 2, 128)])
@pytest.mark.parametrize("pos", [0, 5, 255, 256, 700])
def test_rope_append_attend(ext, bits, q_heads, kv_heads, d, pos):
    """One launch against RoPE in PyTorch + kv_append + kv_decode_attention on a cache that
    already holds `pos` tokens."""
    torch.manual_seed(4)
    t_max = 1024
    width = d if bits == 8 else d // 2
    dt = torch.int8 if bits == 8 else torch.uint8

    def fresh():
        return dict(kc=torch.zeros(kv_heads, t_max, width, dtype=dt, device="cuda"),
                    vc=torch.zeros(kv_heads, t_max, width, dtype=dt, device="cuda"),
                    ks=torch.zeros(kv_heads, t_max, device="cuda"), vs=torch.zeros(kv_heads, t_max, device="cuda"))

    a, b = fresh(), fresh()
    zero = torch.zeros(1, dtype=torch.int32, device="cuda")
    if pos:
        past_k = torch.randn(kv_heads, pos, d).to(torch.bfloat16).cuda()
        past_v = torch.randn(kv_heads, pos, d).to(torch.bfloat16).cuda()
        for c in (a, b):
            ext.kv_append(past_k, past_v, c["kc"], c["vc"], c["ks"], c["vs"], zero, False)
    inv_freq = 1.0 / (500000.0 ** (torch.arange(0, d, 2).float() / d))
    freqs = torch.outer(torch.arange(t_max).float(), inv_freq)
    emb = torch.cat((freqs, freqs), -1)
    cos_t, sin_t = emb.cos().to(torch.bfloat16).cuda(), emb.sin().to(torch.bfloat16).cuda()
    qkv = torch.randn(1, (q_heads + 2 * kv_heads) * d).to(torch.bfloat16).cuda()
    position = torch.tensor([pos], dtype=torch.int32, device="cuda")
    got = ext.kv_rope_append_attend(qkv, cos_t, sin_t, a["kc"], a["vc"], a["ks"], a["vs"], position, d ** -0.5, q_heads)

    q = qkv[0, : q_heads * d].view(q_heads, d)
    k = qkv[0, q_heads * d: (q_heads + kv_heads) * d].view(kv_heads, d)
    v = qkv[0, (q_heads + kv_heads) * d:].view(kv_heads, d)
    q_r, k_r = rope_reference(q, cos_t[pos], sin_t[pos]), rope_reference(k, cos_t[pos], sin_t[pos])
    ext.kv_append(k_r[:, None], v[:, None], b["kc"], b["vc"], b["ks"], b["vs"], position, False)
    ws = torch.zeros(ext.kv_decode_workspace_floats(q_heads, d, t_max), device="cuda")
    length = torch.tensor([pos + 1], dtype=torch.int32, device="cuda")
    want = ext.kv_decode_attention(q_r.contiguous(), b["kc"], b["vc"], b["ks"], b["vs"], ws, length, d ** -0.5)
    for name in ("kc", "vc", "ks", "vs"):
        assert torch.equal(a[name], b[name]), name  # what was appended is identical
    assert got.shape == (1, q_heads * d)
    assert rel_l2(to_np(got).reshape(q_heads, d), to_np(want)) <= 4e-3  # same math, different merge order


def test_argmax_row(ext):
    torch.manual_seed(5)
    for n in (1, 7, 1000, 128256):
        for dtype in (torch.bfloat16, torch.float32):
            x = torch.randn(1, n).to(dtype).cuda()
            assert ext.argmax_row(x).item() == x.float().argmax().item()
    x = torch.zeros(1, 5000, device="cuda", dtype=torch.bfloat16)
    x[0, [17, 4000, 4999]] = 3.0
    assert ext.argmax_row(x).item() == 17  # first of equal maxima
    assert ext.argmax_row(x[:, 1:].contiguous()[:, :3000].contiguous()).item() == 16  # misaligned / short rows too


def test_argmax_advance_does_the_loop_bookkeeping(ext):
    x = torch.randn(1, 5000, device="cuda").to(torch.bfloat16)
    token = torch.zeros(1, dtype=torch.long, device="cuda")
    step64 = torch.tensor([41], dtype=torch.long, device="cuda")
    step32 = torch.tensor([41], dtype=torch.int32, device="cuda")
    for _ in range(2):
        got = ext.argmax_advance(x, token, step64, step32)
    want = x.float().argmax().item()
    assert got.item() == want and token.item() == want and step64.item() == 43 and step32.item() == 43


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("n", [128256, 5000, 37, 8])
def test_argmax_advance_embed_picks_the_same_token_and_hands_over_its_row(ext, dtype, n):
    """The 32-workgroup form against the one-workgroup one and torch: first maximum among ties that fall in
    different slices, the loop's bookkeeping, the winner's embedding row, and a workspace left ready for the
    next call (three calls in a row on different rows)."""
    gen = torch.Generator().manual_seed(n)
    table = torch.randn(n, 64, generator=gen).to(dtype).cuda()
    hidden = torch.zeros(1, 64, dtype=dtype, device="cuda")
    ws = torch.zeros(ext.argmax_workspace_ints(), dtype=torch.int32, device="cuda")
    token = torch.zeros(1, dtype=torch.long, device="cuda")
    step64 = torch.tensor([7], dtype=torch.long, device="cuda")
    step32 = torch.tensor([7], dtype=torch.int32, device="cuda")
    for call in range(3):
        x = torch.randn(1, n, generator=gen).to(dtype)
        if call == 1 and n > 100:   # equal maxima far apart: the first one wins
            x[0, [n // 3, n // 3 + 1, n - 2]] = 9.0
        x = x.cuda()
        got = ext.argmax_advance_embed(x, token, step64, step32, table, hidden, ws)
        want = ext.argmax_row(x).item()
        assert want == x.float().argmax().item() or call == 1
        assert got.item() == want and token.item() == want
        assert step64.item() == 8 + call and step32.item() == 8 + call
        assert torch.equal(hidden[0], table[want])
        assert ws[64].item() == 0   # the arrival counter, behind the 32 + 32 slice results
    # without the hand-off: only the pick and the bookkeeping
    got = ext.argmax_advance_embed(x, token, step64, step32, None, None, ws)
    assert got.item() == want and step64.item() == 11
    with pytest.raises(RuntimeError, match="go together"):
        ext.argmax_advance_embed(x, token, step64, step32, table, None, ws)
    with pytest.raises(RuntimeError, match="workspace"):
        ext.argmax_advance_embed(x, token, step64, step32, None, None, ws[:8])


def test_fused_runtime_equals_the_unfused_one():
    """Whole decode steps on a small model: fused and operation-by-operation runtimes give the
    same logits to the bit (hidden 512: the variance reduction happens to agree), the same
    tokens, and graph replay equals eager."""
    from test_gpu_decode import build_model, quantized_pair

    from llmquant.runtime import LlamaFusedRuntime, LlamaKernelRuntime, kernel_runtime

    _, kernel = quantized_pair(build_model(512, 1024, 3, 8, 2, 4096))
    ids = torch.randint(0, 4096, (1, 40), generator=torch.Generator().manual_seed(1)).cuda()
    plain, fused = LlamaKernelRuntime(kernel, 80, 8), LlamaFusedRuntime(kernel, 80, 8)
    assert isinstance(kernel_runtime(kernel, 80, 8), LlamaFusedRuntime)
    tok = plain.prefill(ids)
    assert torch.equal(tok, fused.prefill(ids))
    for i in range(16):
        logits_p, nxt_p = plain.eager_step(tok, 40 + i)
        logits_f, nxt_f = fused.eager_step(tok, 40 + i)
        assert rel_l2(to_np(logits_f), to_np(logits_p)) <= 2e-2
        assert torch.equal(plain.cache.k_codes[:, :, : 40 + i + 1], fused.cache.k_codes[:, :, : 40 + i + 1]) or i > 0
        tok = nxt_p
    seq_g = LlamaFusedRuntime(kernel, 80, 8).generate(ids, 24, use_graph=True)
    seq_e = LlamaFusedRuntime(kernel, 80, 8).generate(ids, 24, use_graph=False)
    assert torch.equal(seq_g, seq_e)
    # one workgroup per head and several give the same tokens here, and each replays as it runs eagerly
    one = LlamaFusedRuntime(kernel, 80, 8, attn_splits=1)
    many = LlamaFusedRuntime(kernel, 80, 8, attn_splits=5)
    assert fused.attn_splits > 1 and one.attn_splits == 1
    assert torch.equal(one.generate(ids, 24, use_graph=True), one.generate(ids, 24, use_graph=False))
    assert torch.equal(many.generate(ids, 24, use_graph=True), seq_g)


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("q_heads,kv_heads,d", [(32, 8, 64), (8, 2, 128)])
# (32 splits and more: four query heads of a kv head share a workgroup)
@pytest.mark.parametrize("pos,splits", [(0, 8), (5, 8), (63, 2), (64, 3), (700, 8), (2047, 16), (300, 1), (1500, 2),
                                        (0, 32), (77, 32), (2047, 32), (1900, 40)])
def test_split_attention_and_its_merge(ext, bits, q_heads, kv_heads, d, pos, splits):
    """Tokens of a head spread over `splits` workgroups: the cache ends up identical to the
    one-workgroup launch, the merged output agrees with it (another summation order), and the GEMV
    that merges while staging equals merge-then-GEMV bit for bit."""
    torch.manual_seed(6)
    t_max = 2048
    width = d if bits == 8 else d // 2
    dt = torch.int8 if bits == 8 else torch.uint8

    def fresh():
        return dict(kc=torch.zeros(kv_heads, t_max, width, dtype=dt, device="cuda"),
                    vc=torch.zeros(kv_heads, t_max, width, dtype=dt, device="cuda"),
                    ks=torch.zeros(kv_heads, t_max, device="cuda"), vs=torch.zeros(kv_heads, t_max, device="cuda"))

    a, b = fresh(), fresh()
    zero = torch.zeros(1, dtype=torch.int32, device="cuda")
    if pos:
        past_k = torch.randn(kv_heads, pos, d).to(torch.bfloat16).cuda()
        past_v = torch.randn(kv_heads, pos, d).to(torch.bfloat16).cuda()
        for c in (a, b):
            ext.kv_append(past_k, past_v, c["kc"], c["vc"], c["ks"], c["vs"], zero, False)
    # what the cache holds past the position is read ahead of the position by the split kernel and must
    # be dropped: poison it (scales NaN, codes at their extremes)
    for c in (a, b):
        c["ks"][:, pos + 1:] = float("nan")
        c["vs"][:, pos + 1:] = float("nan")
        c["kc"][:, pos + 1:] = 127
        c["vc"][:, pos + 1:] = 127
    table = torch.randn(t_max, d).clamp(-1, 1).to(torch.bfloat16).cuda()
    qkv = torch.randn(1, (q_heads + 2 * kv_heads) * d).to(torch.bfloat16).cuda()
    position = torch.tensor([pos], dtype=torch.int32, device="cuda")
    want = ext.kv_rope_append_attend(qkv, table, table, b["kc"], b["vc"], b["ks"], b["vs"], position, d ** -0.5, q_heads)
    partials = torch.full((ext.kv_attend_partials_floats(q_heads, d, splits),), float("nan"), device="cuda")
    ext.kv_rope_append_attend_split(qkv, table, table, a["kc"], a["vc"], a["ks"], a["vs"], partials, position,
                                    d ** -0.5, q_heads, splits)
    for name in ("kc", "vc"):
        assert torch.equal(a[name], b[name]), name
    for name in ("ks", "vs"):  # (NaN != NaN: compare the bits)
        assert torch.equal(a[name].view(torch.int32), b[name].view(torch.int32)), name
    merged = ext.kv_attend_merge(partials, q_heads, d, splits, torch.bfloat16)
    assert merged.shape == want.shape and torch.isfinite(merged).all()
    assert rel_l2(to_np(merged), to_np(want)) <= 4e-3

    if q_heads * d % 512 == 0:  # a Linear over the attention output, rows of 4 groups or more
        n, k = 256, q_heads * d
        q, s = weights(n, k, bits, head_dim=d if d < 128 else None)
        res = torch.randn(1, n).to(torch.bfloat16).cuda()
        in_head_dim = d if d < 128 else 0
        got = ext.wq_gemv_attn_merge(partials, splits, d, q, s, 0, in_head_dim, res, torch.bfloat16)
        assert torch.equal(got, ext.wq_gemv_fused(merged, q, s, 0, 0, None, 0.0, in_head_dim, res))


def test_split_attention_argument_checks(ext):
    partials = torch.zeros(16, device="cuda")
    q, s = weights(64, 512, 8)
    with pytest.raises(RuntimeError, match="too small"):
        ext.wq_gemv_attn_merge(partials, 8, 64, q, s, 0, 0, None, torch.bfloat16)
    with pytest.raises(RuntimeError, match="whole number of heads"):
        ext.wq_gemv_attn_merge(torch.zeros(4096, device="cuda"), 2, 96, q, s, 0, 0, None, torch.bfloat16)


def test_prompt_pass_with_its_own_attention_and_two_launch_mlp():
    """A 300-token prompt through a model whose MLP is wide enough for the two-launch form (gate|up with
    silu(gate) * up written as down_proj's prepared activation: 3 x 64 tiles) and whose attention goes through
    llmq_prefill_attention, against the same runtime with the MLP as three launches (bit-equal: hidden states of
    every layer, the cache, the token) and with torch's scaled_dot_product_attention for the prompt (floating
    point: the first layer's cache codes equal, the second's within one step of each other, logits of the last position to
    rel-L2 <= 2e-2, the bound the fused and unfused steps are held to)."""
    from test_gpu_decode import build_model, quantized_pair

    from llmquant.runtime import LlamaFusedRuntime, LlamaKernelRuntime

    _, kernel = quantized_pair(build_model(512, 8192, 2, 8, 2, 4096))
    ids = torch.randint(0, 4096, (1, 300), generator=torch.Generator().manual_seed(2)).cuda()
    calls = {"mlp": 0, "attn": 0}

    class Counting(LlamaFusedRuntime):
        def _mlp(self, index, layer, x):
            out = super()._mlp(index, layer, x)
            calls["mlp"] += 1
            return out

    class ThreeLaunchMlp(LlamaFusedRuntime):
        def _mlp(self, index, layer, x):
            return LlamaKernelRuntime._mlp(self, index, layer, x)

    class LibraryAttention(LlamaFusedRuntime):
        PROMPT_ATTENTION_MAX_TOKENS = {}

    fused = Counting(kernel, 320, 8)
    # (the two-launch path is the one that runs: its extension call is made once per layer)
    ext_calls = []
    # (on rows that the norm in front of it left in prepared form: llmq_add_rmsnorm_prepared)
    real_call = fused._ext.wq_gemm_a16_tile_gate_up_silu_prepared
    try:
        fused._ext.wq_gemm_a16_tile_gate_up_silu_prepared = lambda *a, **k: (ext_calls.append(1), real_call(*a, **k))[1]
        tok = fused.prefill(ids)
    finally:
        fused._ext.wq_gemm_a16_tile_gate_up_silu_prepared = real_call
    assert calls["mlp"] == 2 and len(ext_calls) == 2
    three = ThreeLaunchMlp(kernel, 320, 8)
    assert torch.equal(three.prefill(ids), tok)
    for name in ("k_codes", "v_codes", "k_scale", "v_scale"):
        assert torch.equal(getattr(three.cache, name), getattr(fused.cache, name)), name
    logits_fused, _ = fused.eager_step(tok, 300)
    logits_three, _ = three.eager_step(tok, 300)
    assert torch.equal(logits_fused, logits_three)
    library = LibraryAttention(kernel, 320, 8)
    library.prefill(ids)
    logits_library, _ = library.eager_step(tok, 300)
    assert rel_l2(to_np(logits_fused), to_np(logits_library)) <= 2e-2
    assert torch.equal(library.cache.k_codes[0, :, :300], fused.cache.k_codes[0, :, :300])
    step = (library.cache.k_codes[1, :, :300].int() - fused.cache.k_codes[1, :, :300].int()).abs()
    assert float((step <= 1).float().mean()) > 0.99 and int(step.max()) <= 3


def test_decode_step_follows_the_tokens_the_cache_holds_through_two_regimes():
    """A long cache that is mostly empty: below a threshold of cached tokens the step runs the attention launch with
    the short cache's split count, from there on with the many-split form (here: the matrix-core kernel, the cache
    has 12288 rows), each regime with a captured step of its own. Graph replay and eager steps pick the same
    launches at the same positions, so their tokens are equal; a second generation reuses both captured steps."""
    from test_gpu_decode import build_model, quantized_pair

    from llmquant.runtime import LlamaFusedRuntime

    _, kernel = quantized_pair(build_model(512, 1024, 3, 8, 2, 4096))
    ids = torch.randint(0, 4096, (1, 40), generator=torch.Generator().manual_seed(5)).cuda()

    def runtime():
        rt = LlamaFusedRuntime(kernel, 12288, 8)
        assert rt.attn_splits == 32 and rt.regimes is None
        rt.regimes = [(0, 8), (48, 32)]   # (8 heads: the automatic choice has one regime; forced here)
        return rt

    eager, graphed = runtime(), runtime()
    seen = []
    real = eager._ext.kv_rope_append_attend_split
    try:
        eager._ext.kv_rope_append_attend_split = lambda *a: (seen.append((eager.cache.get_seq_length(), a[11])), real(*a))[1]
        out_eager = eager.generate(ids, 24, use_graph=False)
    finally:
        eager._ext.kv_rope_append_attend_split = real
    by_position = dict(seen)
    assert all(by_position[p] == (8 if p < 48 else 32) for p in range(40, 63)), by_position
    out_graphed = graphed.generate(ids, 24, use_graph=True)
    assert torch.equal(out_graphed, out_eager)
    assert sorted(graphed._graphs) == [8, 32]
    kept = dict(graphed._graphs)
    assert torch.equal(graphed.generate(ids, 24, use_graph=True), out_eager)
    assert all(graphed._graphs[k][0] is kept[k][0] for k in kept)   # no step was captured again
    # a prompt that already lies in the long regime starts there
    long_ids = torch.randint(0, 4096, (1, 60), generator=torch.Generator().manual_seed(6)).cuda()
    assert torch.equal(graphed.generate(long_ids, 8, use_graph=True), eager.generate(long_ids, 8, use_graph=False))


def test_regimes_the_fused_runtime_picks():
    """32 query heads on 8 kv heads: caches up to 5120 rows have one regime (8 splits); longer ones go to 16 splits from
    5120 cached tokens and, beyond 16384 rows, to 32 from 16384. An explicit split count is one regime; a model
    without grouped heads keeps the split count that grows with the cache."""
    from test_gpu_decode import build_model, quantized_pair

    from llmquant.runtime import LlamaFusedRuntime

    _, kernel = quantized_pair(build_model(2048, 1024, 1, 32, 8, 4096))
    assert LlamaFusedRuntime(kernel, 769, 8).regimes is None and LlamaFusedRuntime(kernel, 4096, 8).attn_splits == 8
    mid = LlamaFusedRuntime(kernel, 8192, 8)
    assert mid.regimes == [(0, 8), (5120, 16)] and mid.attn_splits == 16
    assert [mid._splits_for(n) for n in (0, 5119, 5120, 8000)] == [8, 8, 16, 16]
    long = LlamaFusedRuntime(kernel, 32768, 8)
    assert long.regimes == [(0, 8), (5120, 16), (16384, 32)] and long.attn_splits == 32
    assert [long._splits_for(n) for n in (100, 6000, 16383, 16384, 32000)] == [8, 16, 16, 32, 32]
    assert LlamaFusedRuntime(kernel, 32768, 8, attn_splits=12).regimes is None
    _, plain = quantized_pair(build_model(512, 1024, 1, 8, 8, 4096))
    assert LlamaFusedRuntime(plain, 8192, 8).regimes is None and LlamaFusedRuntime(plain, 8192, 8).attn_splits == 32
