"""The host-side package (llm-quant_amd/llmquant) behaves like the reference's API: the facts the
reference's CPU tests assert (tests/test_quantization.py, test_grouping.py, test_real_quant.py,
test_packing.py, test_kv_cache.py, test_config.py), re-asserted on this implementation, plus
agreement of its PyTorch arithmetic with the numpy oracle."""

import json
import struct

import numpy as np
import pytest
import torch
import torch.nn as nn

import llmq_oracle as oracle
from llmquant import QuantConfig, QuantizationModifier, oneshot
from llmquant.core import QuantizationArgs, preset_name_to_scheme
from llmquant.core.layout import WeightLayout, layout_for
from llmquant.core.observers import compute_scale, group_view, pad_to_group, ungroup
from llmquant.core.quant_ops import fake_quantize, quantize
from llmquant.core.scheme import GROUP_SIZE, PRESET_SCHEMES, QuantizationScheme
from llmquant.packing import (pack_int4, pack_weight, read_header, read_packed, unpack_int4,
                              unpack_weight, write_packed)
from llmquant.packing.format import ALIGNMENT, MAGIC
from llmquant.quantizers import (AVAILABLE_MODES, KERNEL_MAX_ROWS, FakeQuantCache, FakeQuantLinear,
                                 RealQuantLinear, exact_fp32_matmul, make_cache_factory, pad_activation,
                                 quant_linear_for, quantize_weight)

HEADS, HEAD_DIM, K = 32, 64, 2048


# ---- schemes and config -----------------------------------------------------------------------------

def test_scheme_validation_and_presets():
    with pytest.raises(ValueError, match="requires a positive group_size"):
        QuantizationArgs(num_bits=4, strategy="group")
    with pytest.raises(ValueError, match="only valid for strategy"):
        QuantizationArgs(num_bits=4, strategy="channel", group_size=128)
    assert set(PRESET_SCHEMES) == {"W4A8", "W8A8", "W4A16", "W8A16"}
    assert preset_name_to_scheme("w4a8").weights.num_bits == 4
    assert preset_name_to_scheme("W8A8").input_activations.dynamic
    assert preset_name_to_scheme("W4A16").input_activations is None
    with pytest.raises(ValueError):
        preset_name_to_scheme("W3A8")
    with pytest.raises(Exception):
        preset_name_to_scheme("W4A8").weights.num_bits = 8  # frozen


def test_config_axes_refusals_and_label():
    from llmquant.core.config import normalize_dtype

    assert [normalize_dtype(v) for v in (None, "bf16", "INT4", " int8 ")] == ["bf16", "bf16", "int4", "int8"]
    with pytest.raises(ValueError, match="unknown dtype"):
        normalize_dtype("fp8")
    cfg = QuantConfig(attn_weight="int8", mlp_weight="int4", head_weight="int8", kv_cache="int8")
    assert cfg.describe() == "attn-int8_mlp-int4_head-int8_act-bf16_kv-int8_g128"
    assert cfg.kv_cache_bits == 8 and QuantConfig().kv_cache_bits is None
    assert cfg.scheme("mlp_weight").weights.num_bits == 4 and QuantConfig().scheme("attn_weight") is None
    assert QuantConfig(attn_weight="int4", activation="int8").scheme("attn_weight").input_activations.num_bits == 8
    for bad in (dict(kv_cache="int4"), dict(head_weight="int4"), dict(activation="int4"), dict(group_size=0)):
        with pytest.raises(ValueError):
            QuantConfig(**bad)
    with pytest.raises(ValueError, match="unknown target"):
        cfg.scheme("kv_cache")
    recipe = cfg.to_modifier(mode="kernel")
    assert recipe.mode == "kernel" and recipe.kv_cache_bits == 8 and recipe.scheme is None


class TinyConfig:
    num_hidden_layers = 1
    num_attention_heads = 2
    num_key_value_heads = 2
    hidden_size = K
    head_dim = HEAD_DIM


class TinyLlama(nn.Module):
    def __init__(self):
        super().__init__()
        self.config = TinyConfig()
        self.model = nn.Module()
        self.model.layers = nn.ModuleList([nn.Module()])
        layer = self.model.layers[0]
        layer.self_attn = nn.Module()
        layer.self_attn.q_proj = nn.Linear(K, 256, bias=False)
        layer.self_attn.o_proj = nn.Linear(K, 256, bias=False)
        layer.mlp = nn.Module()
        layer.mlp.down_proj = nn.Linear(K, 256, bias=False)
        self.lm_head = nn.Linear(K, GROUP_SIZE, bias=False)


def test_routing_by_name():
    recipe = QuantConfig(attn_weight="int4", mlp_weight="int4", activation="int8").to_modifier()
    recipe.resolve(TinyLlama())
    assert recipe.head_dim == HEAD_DIM
    o = recipe.scheme_for("model.layers.0.self_attn.o_proj")
    q = recipe.scheme_for("model.layers.0.self_attn.q_proj")
    mlp = recipe.scheme_for("model.layers.0.mlp.down_proj")
    assert o.weights.head_dim == HEAD_DIM and o.input_activations.head_dim == HEAD_DIM
    assert q.weights.head_dim is None and q.weights.out_group == HEAD_DIM and mlp.weights.head_dim is None
    assert mlp.weights.out_group is None and recipe.scheme_for("lm_head") is None
    fused = recipe.scheme_for("model.layers.0.self_attn.qkv_proj")
    assert fused.weights.out_group == HEAD_DIM
    off = QuantConfig(attn_weight="int8", qkv_out_scale_per_head=False).to_modifier()
    off.head_dim = HEAD_DIM
    assert off.scheme_for("model.layers.0.self_attn.q_proj").weights.out_group is None
    fixed = QuantizationModifier(attn_scheme="W4A16", head_dim=8)
    assert fixed.resolve(TinyLlama()).head_dim == 8


def test_apply_swaps_modules_per_mode():
    class Tiny(nn.Module):
        def __init__(self):
            super().__init__()
            self.proj = nn.Linear(GROUP_SIZE, 8, bias=False)
            self.lm_head = nn.Linear(GROUP_SIZE, 4, bias=False)

    model = QuantizationModifier(scheme="W4A8").apply(Tiny())
    assert isinstance(model.proj, FakeQuantLinear) and isinstance(model.lm_head, nn.Linear)
    model = QuantizationModifier(scheme="W4A8", lm_head_scheme="W8A8").apply(Tiny())
    assert isinstance(model.lm_head, FakeQuantLinear) and model.lm_head.scheme.weights.num_bits == 8
    model = oneshot(Tiny(), QuantizationModifier(scheme="W8A16", mode="real"))
    assert isinstance(model.proj, RealQuantLinear)
    assert AVAILABLE_MODES == {"fake", "real", "kernel"}
    with pytest.raises(ValueError, match="unsupported mode"):
        quant_linear_for("int3")
    full = oneshot(TinyLlama(), QuantConfig(attn_weight="int8", mlp_weight="int4", head_weight="int8").to_modifier("real"))
    assert full.model.layers[0].self_attn.o_proj.scheme.weights.head_dim == HEAD_DIM
    assert full.lm_head.scheme.weights.num_bits == 8


def test_kernel_mode_fails_loudly_without_a_gpu():
    if torch.cuda.is_available():
        pytest.skip("this is the no-GPU behaviour")
    from llmquant.hip import load_extension
    from llmquant.quantizers import KernelQuantLinear

    with pytest.raises(RuntimeError, match="CUDA is not available"):
        load_extension()
    with pytest.raises(RuntimeError, match="CUDA is not available"):
        KernelQuantLinear.from_linear(nn.Linear(128, 8, bias=False), preset_name_to_scheme("W8A16"))
    with pytest.raises(ValueError, match="needs a weight scheme"):
        KernelQuantLinear.from_linear(nn.Linear(128, 8), QuantizationScheme(weights=None, input_activations=None))


def test_row_count_routing_of_the_kernel_mode_linear():
    from llmquant.quantizers import FUSED_GEMM_MAX_ROWS, KERNEL_MAX_ROWS
    from llmquant.quantizers.kernel import FUSED_GEMM_MIN_ROWS, FUSED_GEMM_WHOLE_ROWS, fused_gemm_splits

    # the GEMV keeps the one- and two-row cases, the fused GEMM starts inside the GEMV's range
    # (so there is no gap) and ends where the dense branch takes over
    assert 1 < FUSED_GEMM_MIN_ROWS <= KERNEL_MAX_ROWS + 1
    assert FUSED_GEMM_WHOLE_ROWS == FUSED_GEMM_MAX_ROWS == 64
    # the whole-rows form at every row count and row length (gate/up and down_proj of Llama-3-8B: 32 and 112
    # groups per row): it is the faster one everywhere since its activation goes through LDS
    for rows in (3, 16, 17, 64, 100, 128):
        for groups in (16, 32, 63, 64, 112):
            assert not fused_gemm_splits(rows, groups)


def test_narrow_short_weights_keep_the_fused_gemm_up_to_128_rows():
    from llmquant.quantizers.kernel import fused_gemm_takes, tiled_gemm_pays

    # q|k|v and o_proj of Llama-3.2-1B (16 groups a row) and Llama-3-8B's o_proj (4096 x 32 groups)
    for n, g in ((3072, 16), (2048, 16), (4096, 32)):
        assert fused_gemm_takes(3, n, g) and fused_gemm_takes(64, n, g) and fused_gemm_takes(65, n, g) and fused_gemm_takes(128, n, g)
        assert not fused_gemm_takes(129, n, g) and not fused_gemm_takes(2, n, g)
    # wider or longer weights: 64 rows, then the tiled GEMM or the dense branch
    assert fused_gemm_takes(64, 6144, 32) and not fused_gemm_takes(65, 6144, 32)
    assert fused_gemm_takes(64, 16384, 16) and not fused_gemm_takes(100, 16384, 16) and tiled_gemm_pays(100, 16384, 16)
    assert not fused_gemm_takes(100, 2048, 64) and tiled_gemm_pays(100, 2048, 64)
    # a mid-sized weight (Llama-3-8B's q|k|v): one tile of rows goes to the tiled GEMM; more, as long as the estimate
    # says so (at 512 rows the library is ahead: 48.7 us against 46.5 measured)
    assert tiled_gemm_pays(100, 6144, 32) and tiled_gemm_pays(128, 6144, 32) and tiled_gemm_pays(129, 6144, 32)
    assert not tiled_gemm_pays(100, 4096, 32) and not tiled_gemm_pays(100, 3072, 16)
    # beyond 128 rows: by the estimated times of the two branches (measured cases on both sides of the line)
    # short rows on an output that 64 x 128 tiles cover in one round: q|k|v of Llama-3.2-1B at a 512-token prompt
    assert tiled_gemm_pays(512, 3072, 16) and tiled_gemm_pays(192, 3072, 16) and tiled_gemm_pays(512, 4096, 16)
    assert not tiled_gemm_pays(512, 3072, 24) and not tiled_gemm_pays(512, 2048, 32)   # longer rows: the library
    assert not tiled_gemm_pays(1024, 3072, 16) and tiled_gemm_pays(136, 512, 16)   # two rounds; a dozen tiles (12.6 us / 13.8)
    # wide int4 weights: one round of 128 x 256 tiles pays, a half-empty second round does not
    assert tiled_gemm_pays(512, 14336, 32, 4) and not tiled_gemm_pays(640, 14336, 32, 4)
    assert tiled_gemm_pays(512, 16384, 16, 4) and not tiled_gemm_pays(768, 16384, 16, 4)
    assert not tiled_gemm_pays(1024, 14336, 32, 4) and not tiled_gemm_pays(1025, 2048, 64, 4)
    # a weight whose dequantize pass alone is 73 us keeps the tiled GEMM through its second round; long rows are cut
    assert tiled_gemm_pays(512, 28672, 32, 4) and not tiled_gemm_pays(896, 28672, 32, 4)
    assert tiled_gemm_pays(640, 4096, 112, 4) and tiled_gemm_pays(1024, 2048, 64, 4) and tiled_gemm_pays(768, 2048, 64, 4)
    from llmquant.quantizers.kernel import dense_branch_cost, tiled_gemm_cost

    # the estimates against launches measured on an MI355X (us): within a tenth for the tiled GEMM
    for (m, n, g, bits), measured in {(512, 3072, 16, 8): 24.2, (512, 16384, 16, 4): 46.1, (640, 14336, 32, 4): 139.6,
                                      (2048, 14336, 32, 4): 278.5, (128, 14336, 32, 4): 31.7}.items():
        assert abs(tiled_gemm_cost(m, n, g, bits) / measured - 1) <= 0.1, (m, n, g, bits)
    assert abs(dense_branch_cost(512, 28672, 32, 4) / 163.6 - 1) <= 0.1
    assert tiled_gemm_cost(512, 3072, 16, 8, prepared=True) == tiled_gemm_cost(512, 3072, 16, 8) - 3.5


# ---- layout ---------------------------------------------------------------------------------------------

def test_layout_geometry():
    o = layout_for(2048, 2048, QuantizationArgs(4, "group", group_size=128, head_dim=64))
    assert (o.padded_in, o.in_groups, o.scale_rows, o.num_scales) == (4096, 32, 2048, 2048 * 32)
    q = layout_for(2048, 2048, QuantizationArgs(8, "group", group_size=128, out_group=64))
    assert (q.padded_out, q.scale_rows, q.in_groups) == (4096, 32, 16)
    plain = WeightLayout(100, 300, 128)
    assert (plain.padded_in, plain.padded_out, plain.weight_bytes(4)) == (384, 128, 384 * 128 // 2)
    fused = layout_for((32 + 64) * 96, 3072, QuantizationArgs(8, "group", group_size=128, out_group=96))
    assert fused.padded_out == 96 * 128 and fused.scale_rows == 96
    with pytest.raises(ValueError, match="not a multiple of head_dim"):
        WeightLayout(out_features=9217, in_features=3072, group_size=128, out_head_dim=96)
    assert plain.bits_per_real_element(4, 4) > 4


# ---- the PyTorch arithmetic equals the oracle's -----------------------------------------------------------

@pytest.mark.parametrize("dtype,tag", [(torch.float32, "f32"), (torch.bfloat16, "bf16"), (torch.float16, "f16")])
@pytest.mark.parametrize("kwargs", [dict(), dict(head_dim=64), dict(out_group=16)])
def test_fake_quantize_equals_the_oracle(dtype, tag, kwargs):
    torch.manual_seed(0)
    x = (torch.randn(40, 320) * 2).to(dtype)
    for bits in (4, 8):
        args = QuantizationArgs(bits, "group", group_size=128, **kwargs)
        got = fake_quantize(x, args)
        want = oracle.fake_quantize(x.float().numpy(), bits, tag, "group", 128, **kwargs)
        assert got.dtype == dtype and np.array_equal(got.float().numpy(), want)
        assert np.array_equal(compute_scale(x, args).numpy(), oracle.compute_scale(x.float().numpy(), bits, "group", 128, **kwargs))


def test_known_answers_hold_for_the_torch_form():
    assert quantize(torch.tensor([0.5, 1.5, 2.5, -0.5]), torch.tensor(1.0), preset_name_to_scheme("W8A8").input_activations).tolist() == [0.0, 2.0, 2.0, -0.0]
    x = torch.zeros(1, 128)
    x[0, 0] = 6.2982625961
    args = QuantizationArgs(4, "group", group_size=128)
    assert torch.equal(compute_scale(x, args).flatten(), (x.abs().amax() / torch.tensor(7.0)).flatten())
    w = torch.randn(8, 256)
    assert torch.equal(fake_quantize(w, QuantizationArgs(4, "channel")), fake_quantize(w, QuantizationArgs(4, "group", group_size=256)))
    x = torch.randn(4, 64)
    assert torch.equal(fake_quantize(x, QuantizationArgs(4, "group", group_size=128)), fake_quantize(x, QuantizationArgs(4, "group", group_size=64)))
    for k, padded in [(128, 128), (100, 128), (129, 256)]:
        assert pad_to_group(torch.randn(3, k), 128).shape[-1] == padded
    for k, hd in [(K, None), (K, HEAD_DIM), (100, None)]:
        x = torch.randn(2, k)
        assert torch.equal(ungroup(group_view(x, 128, hd), x.shape, 128, hd), x)
    with pytest.raises(ValueError, match="not a multiple of head_dim"):
        group_view(torch.randn(2, 100), 128, 64)


@pytest.mark.parametrize("name", ["W8A16", "W8A8", "W4A16", "W4A8"])
@pytest.mark.parametrize("kwargs", [dict(), dict(head_dim=64), dict(out_group=16)])
def test_real_mode_module_equals_the_oracle(name, kwargs):
    """RealQuantLinear on CPU against oracle.real_linear: equality for A8 (integer sums are
    exact), float noise for A16 (the in-group fp32 summation order is the BLAS's)."""
    from dataclasses import replace

    torch.manual_seed(0)
    linear = nn.Linear(512, 96, bias=True)
    base = preset_name_to_scheme(name)
    act = base.input_activations
    if act is not None and "head_dim" in kwargs:
        act = replace(act, head_dim=kwargs["head_dim"])
    scheme = QuantizationScheme(weights=replace(base.weights, **kwargs), input_activations=act)
    x = torch.randn(5, 512) * 2
    got = RealQuantLinear.from_linear(linear, scheme)(x).detach().numpy()
    canonical, scales = oracle.canonical_weight(linear.weight.detach().numpy(), base.weights.num_bits, 128, **kwargs)
    padded = oracle.pad_activation(x.numpy(), 128, kwargs.get("head_dim"))
    want = oracle.real_linear(padded, canonical, scales, "f32", kwargs.get("out_group"),
                              8 if base.input_activations else None, linear.bias.detach().numpy())
    if base.input_activations:
        assert np.array_equal(got, want)
    else:
        assert np.linalg.norm(got - want) / np.linalg.norm(want) < 1e-6
    q, scale = quantize_weight(linear.weight.detach(), scheme.weights)
    assert q.dtype == torch.int8 and np.array_equal(q.numpy(), oracle.quantize_weight(linear.weight.detach().numpy(), base.weights.num_bits, 128, **kwargs)[0])


def test_real_mode_module_behaviour():
    linear = nn.Linear(512, 64, bias=True)
    nn.init.constant_(linear.bias, 1.5)
    module = RealQuantLinear.from_linear(linear, preset_name_to_scheme("W8A16"))
    assert torch.allclose(module(torch.zeros(3, 512)), linear.bias.expand(3, 64))
    assert module(torch.randn(2, 5, 512)).shape == (2, 5, 64)
    with pytest.raises(ValueError, match="real quant needs a weight scheme"):
        RealQuantLinear.from_linear(linear, QuantizationScheme(weights=None, input_activations=None))
    before = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = True
    try:
        with exact_fp32_matmul():
            assert torch.backends.cuda.matmul.allow_tf32 is False
        assert torch.backends.cuda.matmul.allow_tf32 is True
    finally:
        torch.backends.cuda.matmul.allow_tf32 = before
    assert KERNEL_MAX_ROWS == 4
    flat = torch.randn(3, K)
    assert pad_activation(flat, QuantizationArgs(8, "group", group_size=128, head_dim=64)).shape == (3, 2 * K)
    assert pad_activation(torch.randn(3, 100), QuantizationArgs(8, "group", group_size=128)).shape == (3, 128)


# ---- packing and the file format ---------------------------------------------------------------------------

def test_nibble_packing():
    assert int(pack_int4(torch.tensor([[-3, 5]], dtype=torch.int8))[0, 0]) == 0xD5
    values = torch.arange(-8, 8, dtype=torch.int8).repeat(4, 1)
    assert torch.equal(unpack_int4(pack_int4(values)), values)
    assert pack_weight(values, 4).numel() * 2 == values.numel()
    assert torch.equal(unpack_weight(pack_weight(values, 8), 8), values)
    rnd = torch.randint(-8, 8, (7, 3, 64), dtype=torch.int8)
    assert np.array_equal(pack_int4(rnd).numpy(), oracle.pack_int4(rnd.numpy()))
    for bad in (9, -9):
        with pytest.raises(ValueError, match=r"must be in \[-8, 7\]"):
            pack_int4(torch.tensor([[bad, 0]], dtype=torch.int8))
    with pytest.raises(ValueError, match="must be even"):
        pack_int4(torch.zeros(1, 3, dtype=torch.int8))
    for bits in (2, 16):
        with pytest.raises(ValueError, match="unsupported num_bits"):
            pack_weight(torch.zeros(2, 2, dtype=torch.int8), bits)
        with pytest.raises(ValueError, match="unsupported num_bits"):
            unpack_weight(torch.zeros(2, 2, dtype=torch.uint8), bits)


def test_file_round_trip_alignment_and_rejections(tmp_path):
    tensors = {
        "packed": torch.randint(0, 255, (4, 8), dtype=torch.uint8),
        "codes": torch.randint(-128, 127, (3, 5), dtype=torch.int8),
        "scale": torch.rand(4, 2),
        "norm": torch.randn(16).to(torch.bfloat16),
    }
    path = write_packed(tmp_path / "sub" / "w.bin", tensors, {"model_id": "test"})
    restored, meta = read_packed(path)
    assert meta["model_id"] == "test" and list(restored) == list(tensors)
    for name, tensor in tensors.items():
        assert restored[name].dtype == tensor.dtype and torch.equal(restored[name], tensor), name
    for entry in read_header(path)["tensors"].values():
        assert entry["offset"] % ALIGNMENT == 0
    # byte-for-byte what the oracle's statement of the format produces
    as_np = {n: (str(t.dtype).removeprefix("torch."), t.view(torch.uint16).numpy() if t.dtype == torch.bfloat16 else t.numpy())
             for n, t in tensors.items()}
    assert path.read_bytes() == oracle.packed_file_bytes(as_np, {"model_id": "test"})
    foreign = tmp_path / "not-ours.bin"
    foreign.write_bytes(b"SOMETHING" + b"\0" * 64)
    with pytest.raises(ValueError, match="not a llmquant weight file"):
        read_header(foreign)
    header = json.dumps({"version": 999, "meta": {}, "tensors": {}}).encode()
    future = tmp_path / "future.bin"
    future.write_bytes(MAGIC + struct.pack("<Q", len(header)) + header)
    with pytest.raises(ValueError, match="unsupported file version"):
        read_header(future)
    empty = write_packed(tmp_path / "empty.bin", {}, {"model_id": "none"})
    assert read_packed(empty) == ({}, {"model_id": "none"})


# ---- KV cache (fake mode) -------------------------------------------------------------------------------------

@pytest.mark.parametrize("bits", [4, 8])
def test_fake_quant_cache(bits):
    torch.manual_seed(0)
    shape = (1, 2, 5, HEAD_DIM)
    keys, values = torch.randn(*shape), torch.randn(*shape)
    cache = FakeQuantCache(bits)
    ck, cv = cache.update(keys, values, 0)
    args = QuantizationArgs(bits, "group", group_size=128, dynamic=True)
    assert torch.equal(ck, fake_quantize(keys, args)) and torch.equal(cv, fake_quantize(values, args))
    assert torch.equal(ck, fake_quantize(keys, QuantizationArgs(bits, "group", group_size=HEAD_DIM)))
    assert not torch.equal(ck, keys) and cache._args(keys).group_size == 128
    kept = ck.clone()
    more = torch.randn(1, 2, 2, HEAD_DIM)
    all_k, _ = cache.update(more, more.clone(), 0)
    assert all_k.shape[2] == 7 and torch.equal(all_k[:, :, :5], kept)  # old tokens are not re-quantized
    assert make_cache_factory(None) is None and isinstance(make_cache_factory(bits)(), FakeQuantCache)


def test_verification_plan_and_reconcile_follow_the_report_format():
    """eval/verify.py: baseline, selected, one ablation per out-of-kernel axis that is quantized;
    measured speedup, whether the projection held, and what each ablation recovers."""
    from llmquant import QuantConfig
    from llmquant.eval import PROJECTION_TOLERANCE, latency_row, reconcile, verification_plan

    quant = QuantConfig(attn_weight="int8", mlp_weight="int4", head_weight="int8", kv_cache="int8")
    plan = verification_plan(quant)
    assert [label for label, _ in plan] == ["bf16 baseline", "selected", "selected, kv_cache=bf16"]
    assert plan[0][1] is None and plan[2][1].kv_cache == "bf16" and plan[2][1].mlp_weight == "int4"
    both = verification_plan(QuantConfig(), {"attn_weight": "int8", "mlp_weight": "int8", "head_weight": "bf16",
                                             "activation": "int8", "kv_cache": "int8"})
    assert [label for label, _ in both][2:] == ["selected, kv_cache=bf16", "selected, activation=bf16"]
    assert verification_plan(QuantConfig(mlp_weight="int4"))[-1][0] == "selected"

    lat = {"ttft_ms": 8.0, "decode_tps": 250.0, "cuda_graph": True, "peak_vram_gb": 3.0,
           "latency_prompt_tokens": 512, "latency_new_tokens": 256}
    base = dict(latency_row(None, "kernel", lat), verify_label="bf16 baseline")
    assert base["name"] == "bf16" and base["quantize"] is False and base["latency_mode"] == "kernel"
    assert base["attn_weight"] == "bf16" and base["group_size"] == 128
    sel = dict(latency_row(quant, "kernel", dict(lat, decode_tps=1000.0, ttft_ms=8.4, peak_vram_gb=1.5)),
               verify_label="selected", decode_speedup_projected=2.8)
    assert sel["name"] == "attn-int8_mlp-int4_head-int8_act-bf16_kv-int8_g128" and sel["kv_cache"] == "int8"
    abl = dict(latency_row(plan[2][1], "kernel", dict(lat, decode_tps=1100.0)), verify_label="selected, kv_cache=bf16")
    out = reconcile([base, sel, abl])
    assert out["measured_decode_speedup"] == 4.0 and out["held_up"] is True
    assert out["ttft_ratio"] == pytest.approx(1.05) and out["vram_ratio"] == 0.5
    assert out["attribution"] == [{"axis": "kv_cache", "dtype": "int8", "tps_without_it": 1100.0,
                                   "recovered": 1.1, "costs_decode_pct": pytest.approx(100 / 11)}]
    assert reconcile([base]) == {}
    assert reconcile([base, dict(sel, decode_speedup_projected=4.0 / PROJECTION_TOLERANCE + 0.1)])["held_up"] is False


def test_deployed_cost_of_a_bf16_model_and_the_row_columns():
    """llmquant.eval.deployed_cost on an unquantized model: every Linear and the untied lm_head at two bytes
    per weight, the embedding on disk but not in the per-token traffic, the KV cache per token of context
    (llmquant/core/metrics.py:183-200: 32 KB per token at the Llama-3.2-1B geometry in bf16, 17 KB as int8
    with one fp32 scale per token per head, 9 KB as int4); and the four columns a result row carries."""
    from transformers import LlamaConfig, LlamaForCausalLM

    from llmquant.eval import cost_columns, deployed_cost, kv_cache_bytes_per_token, latency_row

    cfg = LlamaConfig(hidden_size=64, intermediate_size=128, num_hidden_layers=2, num_attention_heads=4,
                      num_key_value_heads=2, head_dim=16, vocab_size=100, tie_word_embeddings=False)
    model = LlamaForCausalLM(cfg)
    linears = 2 * (64 * 64 * 2 + 2 * 32 * 64 + 3 * 64 * 128) + 100 * 64   # q, o, k, v, gate, up, down; lm_head
    norms = (2 * 2 + 1) * 64
    cost = deployed_cost(model, None)
    assert cost["decode_bytes_per_token"] == 2 * (linears + norms)
    assert cost["deployed_bytes"] == 2 * (linears + norms + 100 * 64)
    assert cost["bits_per_element"] == 16.0
    assert cost["kv_bytes_per_token"] == 2 * 2 * 2 * 16 * 2

    class Geometry:
        config = LlamaConfig(hidden_size=2048, num_hidden_layers=16, num_attention_heads=32, num_key_value_heads=8,
                             head_dim=64)

    assert kv_cache_bytes_per_token(Geometry, None) == 32 * 1024
    assert kv_cache_bytes_per_token(Geometry, 8) == 17 * 1024
    assert kv_cache_bytes_per_token(Geometry, 4) == 9 * 1024
    row = latency_row(None, "hf_static_cache_graph", {"ttft_ms": 1.0, "decode_tps": 2.0}, cost=cost)
    assert set(cost_columns(cost)) <= set(row) and row["latency_mode"] == "hf_static_cache_graph"
    assert list(row)[:8] == ["name", "quantize", "attn_weight", "mlp_weight", "head_weight", "activation", "kv_cache",
                             "group_size"]
    tied = LlamaForCausalLM(LlamaConfig(hidden_size=64, intermediate_size=128, num_hidden_layers=1,
                                        num_attention_heads=4, num_key_value_heads=2, head_dim=16, vocab_size=100,
                                        tie_word_embeddings=True))
    shared = deployed_cost(tied, None)
    per_layer = 64 * 64 * 2 + 2 * 32 * 64 + 3 * 64 * 128
    assert shared["deployed_bytes"] == 2 * (per_layer + 3 * 64 + 100 * 64)   # the shared table once
