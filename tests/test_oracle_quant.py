"""Pinning the CPU oracle (oracle/llmq_oracle.py and its C twin) before anything trusts it.

Three kinds of check, chosen so a plausible slip -- reciprocal multiply instead of division,
half-away rounding, a transposed operand, the wrong nibble order, a dropped scale -- fails at
least one: the reference's own inline known answers (tests/golden/known_answers.json), what
the mathematics fixes (exact integer sums, float64 closed forms, invariants, brute force on
tiny inputs), and agreement with independently written code (torch CPU ops, the C oracle).
"""

import ctypes
import json
import pathlib
import struct
import subprocess

import numpy as np
import pytest
import torch

import llmq_oracle as oracle

ROOT = pathlib.Path(__file__).resolve().parent.parent
KAT = json.loads((ROOT / "tests" / "golden" / "known_answers.json").read_text())


# ---- storage types ------------------------------------------------------------------------------

def test_bf16_rounding_known_bit_patterns():
    cases = {
        1.0: 0x3F80, -2.0: 0xC000, 0.0: 0x0000,
        1.00390625: 0x3F80,          # 1 + 2^-8: exactly half way, ties to even (down)
        1.01171875: 0x3F82,          # 1 + 3*2^-8: half way, ties to even (up)
        1.0039063692092896: 0x3F81,  # just above half way
        3.3895313892515355e38: 0x7F7F,  # largest finite bf16
    }
    for value, bits in cases.items():
        assert int(oracle.bf16_bits(np.float32(value)).ravel()[0]) == bits, value
    assert int(oracle.bf16_bits(np.float32(np.nan)).ravel()[0]) == 0x7FC0
    assert int(oracle.bf16_bits(np.float32(3.4e38)).ravel()[0]) == 0x7F80  # rounds up to inf


def test_storage_rounding_agrees_with_torch_casts():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(20000).astype(np.float32) * 10.0 ** rng.integers(-8, 8, 20000),
                        np.array([0.0, -0.0, 1e-40, 65504.0, 65520.0, 1e-8, 3e38], dtype=np.float32)]).astype(np.float32)
    t = torch.from_numpy(x)
    assert np.array_equal(oracle.round_to(x, "bf16"), t.to(torch.bfloat16).float().numpy())
    assert np.array_equal(oracle.round_to(x, "f16").view(np.uint32), t.to(torch.float16).float().numpy().view(np.uint32))
    assert oracle.round_to(x, "f32") is not None and np.array_equal(oracle.round_to(x, "f32"), x)


# ---- scales and codes: the reference's known answers -----------------------------------------------

@pytest.mark.parametrize("bits", [4, 8])
def test_weight_quant_is_per_group_symmetric_and_in_range(bits):
    rng = np.random.default_rng(0)
    w = rng.standard_normal((16, 256)).astype(np.float32)
    scale = oracle.compute_scale(w, bits, "group", 128)
    q = oracle.quantize(oracle.group_view(w, 128), scale, bits)
    qmax = 2 ** (bits - 1) - 1
    assert list(scale.shape) == KAT["scale_shape"]["scale_shape"]
    assert np.array_equal(q, np.round(q)) and q.min() >= -qmax - 1 and q.max() <= qmax
    assert np.array_equal(np.abs(q).max(axis=-1), np.full((16, 2), float(qmax)))  # abs-max -> +-qmax


def test_rounding_is_half_to_even():
    k = KAT["half_to_even"]
    q = oracle.quantize(np.array(k["x"], dtype=np.float32), np.float32(k["scale"]), k["bits"])
    assert q.tolist() == k["q"]
    assert np.signbit(q[3])  # -0.5 rounds to negative zero, like torch.round


def test_scale_uses_true_division():
    k = KAT["true_division"]
    x = np.zeros((1, 128), dtype=np.float32)
    x[0, 0] = k["amax"]
    got = oracle.compute_scale(x, 4, "group", 128).ravel()[0]
    want = np.float32(k["amax"]) / np.float32(k["qmax"])
    wrong = np.float32(k["amax"]) * (np.float32(1.0) / np.float32(k["qmax"]))
    assert got == want
    assert want != wrong  # the constant was chosen so the two differ: the check has teeth
    # and against torch's division of a tensor by a tensor
    assert got == (torch.tensor(k["amax"]) / torch.tensor(7.0)).item()


def test_shapes_from_the_reference_tests():
    assert list(oracle.compute_scale(np.zeros((2, 5, 512), np.float32), 8, "group", 128).shape) == KAT["act_scale_shape"]["scale_shape"]
    assert list(oracle.compute_scale(np.ones((4, 100), np.float32), 8, "group", 128).shape) == KAT["tail_padding"]["scale_shape"]
    for k, padded in KAT["pad_sizes"]["cases"]:
        assert oracle.pad_to_group(np.zeros((3, k), np.float32), 128).shape[-1] == padded
    x = np.ones((4, 2048), np.float32)
    assert list(oracle.compute_scale(x, 4, "group", 128).shape) == KAT["head_scale_shapes"]["flat"]
    assert list(oracle.compute_scale(x, 4, "group", 128, head_dim=64).shape) == KAT["head_scale_shapes"]["per_head"]


def test_eps_floor_and_extremes():
    assert oracle.compute_scale(np.zeros((1, 128), np.float32), 8, "group", 128).ravel()[0] == np.float32(1e-8)
    for fill in (0.0, 1e-9, 3e38):
        x = np.full((4, 128), fill, dtype=np.float32)
        out = oracle.fake_quantize(x, 8, "f32", "group", 128)
        assert np.all(np.isfinite(out))
    assert np.all(oracle.fake_quantize(np.full((1, 128), 1e-9, np.float32), 8, "f32", "group", 128) == 0)


def test_tie_ramp_matches_a_by_hand_statement():
    """arange(512).reshape(4,128) - 256 + 0.5: every x/scale lands on or near a tie."""
    x = (np.arange(512, dtype=np.float32).reshape(4, 128) - 256 + 0.5)
    got = oracle.fake_quantize(x, 8, "f32", "group", 128)
    for r in range(4):
        amax = np.abs(x[r]).max()
        s = np.float32(amax) / np.float32(127)
        for c in range(128):
            q = float(np.rint(np.float32(x[r, c]) / s))  # numpy rint is half-to-even
            assert got[r, c] == np.float32(np.float32(min(max(q, -128), 127)) * s)


# ---- invariants ------------------------------------------------------------------------------------

def test_channel_strategy_is_group_of_the_whole_row():
    rng = np.random.default_rng(0)
    w = rng.standard_normal((8, 256)).astype(np.float32)
    a = oracle.fake_quantize(w, 4, "f32", "channel")
    b = oracle.fake_quantize(w, 4, "f32", "group", 256)
    assert np.array_equal(a, b)
    assert np.array_equal(oracle.compute_scale(w, 4, "channel"), oracle.compute_scale(w, 4, "group", 256)[:, 0])


@pytest.mark.parametrize("bits", [4, 8])
def test_padding_is_numerically_free(bits):
    rng = np.random.default_rng(0)
    x = rng.standard_normal((4, 64)).astype(np.float32)
    assert np.array_equal(oracle.fake_quantize(x, bits, "f32", "group", 128),
                          oracle.fake_quantize(x, bits, "f32", "group", 64))


def test_group_view_round_trips_and_matches_brute_force():
    rng = np.random.default_rng(1)
    for k, head_dim in [(2048, None), (2048, 64), (100, None), (192, 96)]:
        x = rng.standard_normal((2, k)).astype(np.float32)
        view = oracle.group_view(x, 128, head_dim)
        assert view.shape[-1] == 128
        assert np.array_equal(oracle.ungroup(view, x.shape, 128, head_dim), x)
    # brute force: element (row, k) of a head-split view
    x = rng.standard_normal((3, 256)).astype(np.float32)
    view = oracle.group_view(x, 128, 64)  # 4 heads of 64, each padded to 128
    for row in range(3):
        for head in range(4):
            for d in range(128):
                want = x[row, head * 64 + d] if d < 64 else 0.0
                assert view[row, head, d] == want
    with pytest.raises(ValueError, match="not a multiple of head_dim"):
        oracle.group_view(np.zeros((2, 100), np.float32), 128, 64)


def test_out_block_scales_are_shared_by_a_tile_of_rows():
    rng = np.random.default_rng(2)
    w = rng.standard_normal((10, 256)).astype(np.float32)  # 10 rows, tiles of 4 -> padded to 12
    scale = oracle.compute_scale(w, 8, "group", 128, out_group=4)
    assert scale.shape == (3, 1, 2, 1)
    for tile in range(3):
        rows = w[tile * 4: tile * 4 + 4]
        for g in range(2):
            amax = np.abs(rows[:, g * 128:(g + 1) * 128]).max()
            assert scale[tile, 0, g, 0] == np.float32(amax) / np.float32(127)
    q, _ = oracle.quantize_weight(w, 8, 128, out_group=4)
    assert q.shape == w.shape and q.dtype == np.int8


def test_fake_quantize_agrees_with_a_torch_restatement():
    """Same three lines written with torch CPU ops (a different library's division, rounding
    and bf16 cast)."""
    torch.manual_seed(0)
    for dtype, tag in ((torch.float32, "f32"), (torch.bfloat16, "bf16"), (torch.float16, "f16")):
        x = (torch.randn(37, 384) * 3).to(dtype)
        for bits in (4, 8):
            qmax = 2 ** (bits - 1) - 1
            g = x.float().reshape(37, 3, 128)
            s = (g.abs().amax(-1, keepdim=True) / torch.tensor(float(qmax))).clamp(min=1e-8)
            want = (torch.clamp(torch.round(g / s), -qmax - 1, qmax) * s).reshape(37, 384).to(dtype)
            got = oracle.fake_quantize(x.float().numpy(), bits, tag, "group", 128)
            assert np.array_equal(got, want.float().numpy()), (dtype, bits)


# ---- weights and the real-mode forward ----------------------------------------------------------------

def test_quantize_weight_facts():
    rng = np.random.default_rng(0)
    w = rng.standard_normal((256, 512)).astype(np.float32) * 0.05
    q, scale = oracle.quantize_weight(w, 4)
    assert q.dtype == np.int8 and q.shape == w.shape and q.min() >= -8 and q.max() <= 7
    assert scale.shape == (256, 4, 1)
    for args in (dict(head_dim=64), dict(out_group=64)):
        q, scale = oracle.quantize_weight(w, 4, 128, **args)
        assert q.shape == w.shape and q.min() >= -8 and q.max() <= 7 and scale.size < w.size
    canonical, flat = oracle.canonical_weight(w, 8, 128, head_dim=64)
    assert canonical.shape == (256, 8, 128) and flat.shape == (256, 8)
    assert np.all(canonical[:, :, 64:] == 0)  # the padded half of every head group


def test_group_partial_sums_are_exact_in_fp32():
    k = KAT["group_sum_exact"]
    assert 128 * 127 * 127 == k["bound"] < k["limit"] == 2 ** 24
    a = np.full((8, 128), 127.0, dtype=np.float32)
    b = np.full((128, 16), 127.0, dtype=np.float32)
    b[:, ::2] = -127.0
    assert np.array_equal(a @ b, (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32))


@pytest.mark.parametrize("act_bits", [None, 8])
@pytest.mark.parametrize("bits", [4, 8])
def test_real_linear_against_brute_force(bits, act_bits):
    """Tiny case, python loops, int64 / float64 arithmetic."""
    rng = np.random.default_rng(3)
    w = rng.standard_normal((5, 256)).astype(np.float32) * 0.1
    x = rng.standard_normal((3, 256)).astype(np.float32)
    canonical, scales = oracle.canonical_weight(w, bits)
    got = oracle.real_linear(x, canonical, scales, "f32", None, act_bits)
    want = np.zeros((3, 5), dtype=np.float32)
    for m in range(3):
        for n in range(5):
            acc = np.float32(0)
            for g in range(2):
                xs = x[m, g * 128:(g + 1) * 128]
                if act_bits:
                    sx = max(np.float32(np.abs(xs).max()) / np.float32(127), np.float32(1e-8))
                    a = [int(min(max(np.rint(np.float32(v) / sx), -128), 127)) for v in xs]
                    total = sum(int(a[k]) * int(canonical[n, g, k]) for k in range(128))
                    part = np.float32(total) * scales[n, g]
                    part = np.float32(part) * np.float32(sx)
                else:
                    total = sum(float(xs[k]) * float(canonical[n, g, k]) for k in range(128))
                    part = np.float32(np.float32(total) * scales[n, g])
                acc = np.float32(acc + part)
            want[m, n] = acc
    assert np.array_equal(got, want)


@pytest.mark.parametrize("name,bits,act", [("W8A16", 8, None), ("W8A8", 8, 8), ("W4A16", 4, None), ("W4A8", 4, 8)])
def test_real_tracks_fake(name, bits, act):
    """Closer to each other than either is to the unquantized product (reference
    tests/test_real_quant.py:33-47)."""
    rng = np.random.default_rng(0)
    w = (rng.standard_normal((256, 512)) / np.sqrt(512)).astype(np.float32)
    x = (rng.standard_normal((32, 512)) * 2).astype(np.float32)
    canonical, scales = oracle.canonical_weight(w, bits)
    real = oracle.real_linear(x, canonical, scales, "f32", None, act)
    xq = oracle.fake_quantize(x, act, "f32", "group", 128) if act else x
    fake = xq @ oracle.fake_quantize(w, bits, "f32", "group", 128).T
    exact = x @ w.T
    assert np.abs(real - fake).mean() < np.abs(fake - exact).mean()
    assert np.abs(real - exact).mean() <= np.abs(fake - exact).mean() * 1.01


def test_real_linear_reduces_to_the_closed_form_and_to_the_dense_weight():
    rng = np.random.default_rng(4)
    w = rng.standard_normal((64, 512)).astype(np.float32) * 0.02
    x = oracle.round_to(rng.standard_normal((2, 512)).astype(np.float32), "bf16")
    for args in (dict(), dict(head_dim=64), dict(out_group=16)):
        canonical, scales = oracle.canonical_weight(w, 8, 128, **args)
        padded = oracle.pad_activation(x, 128, args.get("head_dim"))
        real = oracle.real_linear(padded, canonical, scales, "f32", args.get("out_group"))
        exact = oracle.gemv_float64(padded, canonical, scales, args.get("out_group"))
        dense = padded.astype(np.float64) @ oracle.dequantized_weight(canonical, scales, "f32", args.get("out_group")).astype(np.float64).T
        assert np.linalg.norm(real - exact) / np.linalg.norm(exact) < 1e-6
        assert np.linalg.norm(dense - exact) / np.linalg.norm(exact) < 1e-6
        # and the dequantized weight is the fake-quantized weight
        fq = oracle.fake_quantize(w, 8, "f32", "group", 128, **args)
        dq = oracle.dequantized_weight(canonical, scales, "f32", args.get("out_group"))
        assert np.array_equal(oracle.ungroup(dq.reshape(canonical.shape), w.shape, 128, args.get("head_dim")), fq)


def test_bias_and_output_rounding():
    rng = np.random.default_rng(5)
    w = rng.standard_normal((16, 128)).astype(np.float32)
    canonical, scales = oracle.canonical_weight(w, 8)
    out = oracle.real_linear(np.zeros((2, 128), np.float32), canonical, scales, "bf16", bias=np.full(16, 1.5, np.float32))
    assert np.all(out == 1.5)


# ---- packing -------------------------------------------------------------------------------------------

def test_nibble_packing_known_answer_and_round_trip():
    k = KAT["nibble_example"]
    assert int(oracle.pack_int4(np.array([k["values"]], dtype=np.int8))[0, 0]) == k["byte"] == 0xD5
    values = np.tile(np.arange(-8, 8, dtype=np.int8), (4, 1))
    packed = oracle.pack_int4(values)
    assert packed.dtype == np.uint8 and packed.size * 2 == values.size
    assert np.array_equal(oracle.unpack_int4(packed), values)
    for lo in range(-8, 8):          # exhaustive over every byte
        for hi in range(-8, 8):
            byte = int(oracle.pack_int4(np.array([[lo, hi]], dtype=np.int8))[0, 0])
            assert byte == ((lo + 8) | ((hi + 8) << 4))
    with pytest.raises(ValueError, match="must be even"):
        oracle.pack_int4(np.zeros((1, 3), dtype=np.int8))
    for bad in (9, -9):
        with pytest.raises(ValueError, match=r"must be in \[-8, 7\]"):
            oracle.pack_int4(np.array([[bad, 0]], dtype=np.int8))


def test_packed_file_layout():
    tensors = {
        "a": ("uint8", np.arange(3, dtype=np.uint8)),
        "s": ("float32", np.array([[1.0, 2.0]], dtype=np.float32)),
        "n": ("bfloat16", oracle.bf16_bits(np.array([1.0, -2.0, 0.5], dtype=np.float32))),
    }
    blob = oracle.packed_file_bytes(tensors, {"model_id": "test"})
    assert blob[:8] == b"LLMQUANT"
    (length,) = struct.unpack("<Q", blob[8:16])
    header = json.loads(blob[16:16 + length])
    assert header["version"] == 1 and header["meta"] == {"model_id": "test"}
    assert list(header["tensors"]) == ["a", "s", "n"]
    data = blob[16 + length:]
    for name, (dtype, array) in tensors.items():
        entry = header["tensors"][name]
        assert entry["offset"] % 64 == 0 and entry["dtype"] == dtype and entry["shape"] == list(array.shape)
        assert data[entry["offset"]: entry["offset"] + entry["nbytes"]] == array.tobytes()
    assert header["tensors"]["s"]["offset"] == 64 and header["tensors"]["n"]["offset"] == 128


# ---- KV cache -------------------------------------------------------------------------------------------

@pytest.mark.parametrize("bits", [4, 8])
def test_kv_quant_is_fake_quantize_per_token_per_head(bits):
    rng = np.random.default_rng(0)
    k = oracle.round_to(rng.standard_normal((1, 2, 5, 64)).astype(np.float32), "bf16")
    codes, scale = oracle.kv_quant(k, bits)
    assert codes.shape == k.shape and scale.shape == (1, 2, 5)
    stored = oracle.kv_dequant(codes, scale, "bf16")
    assert np.array_equal(stored, oracle.fake_quantize(k, bits, "bf16", "group", 128))
    assert np.array_equal(stored, oracle.fake_quantize(k, bits, "bf16", "group", 64))
    assert not np.array_equal(stored, k)


def test_attention_reduces_to_a_uniform_average():
    """All-equal scores -> the output is the mean of V; one dominant key -> that key's V."""
    v = np.arange(2 * 6 * 4, dtype=np.float32).reshape(2, 6, 4)
    q = np.zeros((4, 4), dtype=np.float32)
    out = oracle.gqa_decode_attention(q, np.ones((2, 6, 4), np.float32), v, 0.5, "f32")
    assert np.allclose(out[0], v[0].mean(0)) and np.allclose(out[3], v[1].mean(0))
    k = np.zeros((2, 6, 4), np.float32)
    k[:, 2, 0] = 100.0
    q[:, 0] = 1.0
    out = oracle.gqa_decode_attention(q, k, v, 1.0, "f32")
    assert np.allclose(out[1], v[0, 2]) and np.allclose(out[2], v[1, 2])


def test_attention_matches_the_library_routines_the_reference_delegates_to():
    """The reference hands attention to transformers (LlamaAttention -> eager_attention_forward, or
    torch's scaled_dot_product_attention): the oracle must agree with both on grouped-query inputs
    where every kv head differs, at a scale other than 1 and with unequal head counts, so a wrong
    head-to-kv-head map (h % kv_heads instead of h // rep), a dropped scale or a transposed operand
    shows. fp32 library arithmetic against the float64 oracle: 1e-5."""
    import types

    import torch
    from transformers.models.llama.modeling_llama import eager_attention_forward

    rng = np.random.default_rng(3)
    hq, hkv, t, d = 12, 3, 37, 16
    q = rng.standard_normal((hq, d)).astype(np.float32)
    k = rng.standard_normal((hkv, t, d)).astype(np.float32) * 2.0
    v = rng.standard_normal((hkv, t, d)).astype(np.float32)
    scale = 0.31
    mine = oracle.gqa_decode_attention(q, k, v, scale, "f32")

    tq, tk, tv = torch.from_numpy(q)[None, :, None, :], torch.from_numpy(k)[None], torch.from_numpy(v)[None]
    module = types.SimpleNamespace(num_key_value_groups=hq // hkv, training=False)
    eager, _ = eager_attention_forward(module, tq, tk, tv, None, scale)  # [1, 1, Hq, D]
    assert np.allclose(mine, eager[0, 0].numpy(), rtol=1e-5, atol=1e-5)
    sdpa = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, scale=scale, enable_gqa=True)
    assert np.allclose(mine, sdpa[0, :, 0].numpy(), rtol=1e-5, atol=1e-5)
    # the wrong grouping is far outside that tolerance on these inputs
    wrong = oracle.gqa_decode_attention(q, k[[0, 1, 2] * 4][:hq].reshape(hq, t, d), v[[0, 1, 2] * 4][:hq].reshape(hq, t, d),
                                        scale, "f32")
    assert not np.allclose(wrong, eager[0, 0].numpy(), rtol=1e-2, atol=1e-2)


def _bf16_ulps(a, b):
    ia = (np.ascontiguousarray(a, dtype=np.float32).view(np.uint32) >> 16).astype(np.int64)
    ib = (np.ascontiguousarray(b, dtype=np.float32).view(np.uint32) >> 16).astype(np.int64)
    ia = np.where(ia & 0x8000, 0x8000 - ia, ia)
    ib = np.where(ib & 0x8000, 0x8000 - ib, ib)
    return np.abs(ia - ib)


def test_decoder_layer_elementwise_steps_match_the_library_modules():
    """llama_rmsnorm / llama_gated_act / llama_residual_add against transformers' own LlamaRMSNorm and
    LlamaMLP (driven with identity projections) and torch's 16-bit adds, on the CPU. A rounding point
    moved (fp32 product kept past the cast, the weight applied before the cast, silu left unrounded)
    fails the equality; the variance's summation order may move a normalised value by one unit of the
    last place at most, and rarely."""
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaMLP, LlamaRMSNorm

    torch.manual_seed(0)
    for dtype, tag in ((torch.bfloat16, "bf16"), (torch.float16, "f16"), (torch.float32, "f32")):
        x = (torch.randn(3, 2048) * 3).to(dtype)
        norm = LlamaRMSNorm(2048, eps=1e-5).to(dtype)
        with torch.no_grad():
            norm.weight.copy_((1 + 0.1 * torch.randn(2048)).to(dtype))
            theirs = norm(x).float().numpy()
        mine = oracle.llama_rmsnorm(x.float().numpy(), norm.weight.detach().float().numpy(), 1e-5, tag)
        if tag == "bf16":
            ulps = _bf16_ulps(mine, theirs)
            assert ulps.max() <= 1 and (ulps == 0).mean() > 0.999
        else:
            np.testing.assert_allclose(mine, theirs, rtol=2e-3 if tag == "f16" else 1e-6, atol=0)
            assert (mine == theirs).mean() > 0.99
        gate, up = (torch.randn(3, 512) * 2).to(dtype), torch.randn(3, 512).to(dtype)
        cfg = LlamaConfig(hidden_size=512, intermediate_size=512, hidden_act="silu")
        mlp = LlamaMLP(cfg).to(dtype)
        with torch.no_grad():
            theirs = (mlp.act_fn(gate) * up).float().numpy()
        mine = oracle.llama_gated_act(gate.float().numpy(), up.float().numpy(), tag)
        if tag == "f32":
            np.testing.assert_allclose(mine, theirs, rtol=1e-6, atol=1e-12)
        else:
            assert np.array_equal(mine, theirs)
        a, b = torch.randn(3, 512).to(dtype), torch.randn(3, 512).to(dtype)
        assert np.array_equal(oracle.llama_residual_add(a.float().numpy(), b.float().numpy(), tag),
                              (a + b).float().numpy())
    # closed forms: a constant row normalises to +-weight (eps = 0), silu(0) * up = 0
    w = np.linspace(0.5, 1.5, 64, dtype=np.float32)
    assert np.array_equal(oracle.llama_rmsnorm(np.full((1, 64), -4.0, np.float32), w, 0.0, "f32"), -w[None])
    assert np.array_equal(oracle.llama_gated_act(np.zeros((1, 8), np.float32), np.ones((1, 8), np.float32)), np.zeros((1, 8)))
    # a rounding point moved must show: the weight applied in fp32 before the cast differs from the library
    x = (torch.randn(4, 2048) * 3).to(torch.bfloat16)
    wt = (1 + 0.1 * torch.randn(2048)).to(torch.bfloat16)
    xf = x.float().numpy()
    inv = 1.0 / np.sqrt((xf.astype(np.float64) ** 2).mean(-1, keepdims=True) + 1e-5)
    moved = oracle.round_to((wt.float().numpy() * (xf * inv)).astype(np.float32), "bf16")
    assert (moved != oracle.llama_rmsnorm(xf, wt.float().numpy(), 1e-5, "bf16")).mean() > 0.05


def test_prompt_attention_is_the_decode_attention_of_every_prefix_and_the_library_routine():
    """The causal form, pinned three ways: row i equals the one-token attention of query i over keys 0..i
    (the function above, itself pinned against transformers); it equals torch's scaled_dot_product_attention
    with is_causal and enable_gqa, the call the reference's prompt pass ends in (fp32 library arithmetic
    against float64: 1e-5), on unequal head counts, a scale other than 1 and kv heads that all differ; and a mask
    turned the wrong way round (queries seeing the future) is far outside that tolerance."""
    import torch

    rng = np.random.default_rng(8)
    t, hq, hkv, d = 23, 6, 2, 16
    q = rng.standard_normal((t, hq, d)).astype(np.float32)
    k = rng.standard_normal((hkv, t, d)).astype(np.float32) * 1.5
    v = rng.standard_normal((hkv, t, d)).astype(np.float32)
    scale = 0.37
    mine = oracle.gqa_prompt_attention(q, k, v, scale)
    assert mine.shape == (t, hq * d) and mine.dtype == np.float64
    for i in (0, 1, 7, t - 1):
        row = oracle.gqa_decode_attention(q[i], k[:, : i + 1], v[:, : i + 1], scale, "f32")
        assert np.allclose(mine[i].reshape(hq, d), row, rtol=1e-6, atol=1e-6)
    assert np.array_equal(mine[0].reshape(hq, d)[0], v[0, 0].astype(np.float64))
    sdpa = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(q).transpose(0, 1)[None], torch.from_numpy(k)[None], torch.from_numpy(v)[None],
        is_causal=True, scale=scale, enable_gqa=True)[0].transpose(0, 1).reshape(t, hq * d).numpy()
    assert np.allclose(mine, sdpa, rtol=1e-5, atol=1e-5)
    backwards = oracle.gqa_prompt_attention(q[::-1], k[:, ::-1], v[:, ::-1], scale)[::-1]
    assert not np.allclose(backwards, sdpa, rtol=1e-2, atol=1e-2)


# ---- the C oracle says the same ----------------------------------------------------------------------------

@pytest.fixture(scope="module")
def c_oracle():
    lib = ROOT / "oracle" / "libllmq_oracle.so"
    if not lib.exists():
        subprocess.run(["make", "-C", str(ROOT / "oracle")], check=True, capture_output=True)
    return ctypes.CDLL(str(lib))


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def test_c_oracle_fake_quant_is_bit_identical(c_oracle):
    rng = np.random.default_rng(0)
    x = (rng.standard_normal((33, 512)) * 3).astype(np.float32)
    for bits in (4, 8):
        out = np.empty_like(x)
        scale = np.empty(33 * 4, dtype=np.float32)
        c_oracle.llmq_oracle_fake_quant_f32(_ptr(x), _ptr(out), _ptr(scale), ctypes.c_int64(33 * 4), 128, bits)
        assert np.array_equal(out.view(np.uint32), oracle.fake_quantize(x, bits, "f32", "group", 128).view(np.uint32))
        assert np.array_equal(scale, oracle.compute_scale(x, bits, "group", 128).ravel())
        xb = oracle.bf16_bits(x)
        outb = np.empty_like(xb)
        c_oracle.llmq_oracle_fake_quant_bf16(_ptr(xb), _ptr(outb), None, ctypes.c_int64(33 * 4), 128, bits)
        want = oracle.fake_quantize(oracle.bf16_from_bits(xb).reshape(x.shape), bits, "bf16", "group", 128)
        assert np.array_equal(outb, oracle.bf16_bits(want))


@pytest.mark.parametrize("packed", [0, 1])
def test_c_oracle_gemv_and_a8_gemm(c_oracle, packed):
    rng = np.random.default_rng(1)
    bits = 4 if packed else 8
    w = rng.standard_normal((48, 384)).astype(np.float32) * 0.03
    x = oracle.round_to(rng.standard_normal((3, 384)).astype(np.float32), "bf16")
    canonical, scales = oracle.canonical_weight(w, bits, 128, out_group=16)
    stored = oracle.pack_int4(canonical) if packed else canonical
    out = np.empty((3, 48), dtype=np.float32)
    c_oracle.llmq_oracle_real_gemv_bf16(_ptr(oracle.bf16_bits(x)), _ptr(stored), _ptr(scales), _ptr(out), 3, 48, 3, 128, 16, packed)
    exact = oracle.gemv_float64(x, canonical, scales, 16)
    assert np.linalg.norm(out - exact) / np.linalg.norm(exact) < 1e-6
    # A8: integer sums are exact, so the two oracles must agree to the bit
    a, sx = oracle.quant_group_codes(x, 8, 128)
    c_oracle.llmq_oracle_real_gemm_a8(_ptr(a), _ptr(np.ascontiguousarray(sx)), _ptr(stored), _ptr(scales), _ptr(out), 3, 48, 3, 128, 16, packed)
    want = oracle.real_linear(x, canonical, scales, "f32", 16, 8)
    assert np.array_equal(out, want)
