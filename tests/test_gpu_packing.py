"""Packed-file save/load of kernel-mode layers and models (reference tests/test_packing.py:104-223)."""

import json

import numpy as np
import pytest
import torch
import torch.nn as nn

import llmq_oracle as oracle
from conftest import to_np

pytestmark = pytest.mark.gpu
GROUP = 128


def kernel_layer(name, in_f=4 * GROUP, out_f=GROUP, bias=False):
    from llmquant.core.scheme import preset_name_to_scheme
    from llmquant.quantizers import KernelQuantLinear

    linear = nn.Linear(in_f, out_f, bias=bias).cuda().to(torch.bfloat16)
    return linear, KernelQuantLinear.from_linear(linear, preset_name_to_scheme(name))


@pytest.mark.parametrize("name", ["W4A16", "W8A16"])
def test_a_quantized_layer_round_trips_bit_exactly(tmp_path, name):
    from llmquant.packing import read_packed, save_packed_model, unpack_weight

    torch.manual_seed(0)
    linear, module = kernel_layer(name)
    model = nn.Module()
    model.proj = module
    path = save_packed_model(model, tmp_path / "layer.bin", "test/model")
    tensors, meta = read_packed(path)
    spec = meta["layers"]["proj"]
    bits = spec["weights"]["num_bits"]
    restored = unpack_weight(tensors["proj.qweight"], bits).reshape(spec["canonical_shape"])
    assert torch.equal(restored.cuda(), module.qweight) and torch.equal(tensors["proj.wscale"].cuda(), module.wscale)
    # and the bytes are what the oracle says the file holds for this weight
    canonical, scales = oracle.canonical_weight(to_np(linear.weight), bits)
    stored = oracle.pack_int4(canonical) if bits == 4 else canonical
    assert np.array_equal(tensors["proj.qweight"].numpy(), stored)
    assert tensors["proj.qweight"].dtype == (torch.uint8 if bits == 4 else torch.int8)
    assert np.array_equal(tensors["proj.wscale"].numpy(), scales)
    assert spec == {"in_features": 4 * GROUP, "out_features": GROUP, "canonical_shape": [GROUP, 4, GROUP],
                    "weights": {"num_bits": bits, "strategy": "group", "group_size": 128, "head_dim": None,
                                "out_group": None, "symmetric": True, "dynamic": False},
                    "input_activations": None, "bias": False}


def test_only_stored_tensors_are_written_and_describe_reads_the_header(tmp_path):
    from llmquant.packing import describe_packed, packed_dtypes, read_header, save_packed_model

    torch.manual_seed(0)
    model = nn.Module()
    _, model.lm_head = kernel_layer("W8A16", GROUP, GROUP)
    path = save_packed_model(model, tmp_path / "m.bin", "test/model", kv_cache_bits=8)
    header = read_header(path)
    assert set(header["tensors"]) == {"lm_head.qweight", "lm_head.wscale"}
    assert list(header["meta"]) == ["model_id", "layers", "experts", "non_persistent_buffers", "kv_cache_bits"]
    summary = describe_packed(path)
    assert summary["model_id"] == "test/model" and summary["quantized_layers"] == 1 and summary["bytes"] > 0
    dtypes = packed_dtypes(path)
    assert dtypes == {"attn_weight": "bf16", "mlp_weight": "bf16", "head_weight": "int8", "kv_cache": "int8",
                      "activation": "bf16"}
    mixed = nn.Module()
    mixed.model = nn.Module()
    mixed.model.layers = nn.ModuleList([nn.Module(), nn.Module()])
    for i, name in enumerate(("W4A16", "W8A16")):
        mixed.model.layers[i].mlp = nn.Module()
        _, mixed.model.layers[i].mlp.gate_proj = kernel_layer(name, GROUP, GROUP)
    assert packed_dtypes(save_packed_model(mixed, tmp_path / "mixed.bin", "test/model"))["mlp_weight"] == "mixed"


def test_whole_model_round_trip_generates_the_same_tokens(tmp_path):
    """Quantize a random-init Llama, save, load from the file (config passed explicitly: no hub),
    and decode: identical logits, 4-bit layers still packed on the device, and a load peak
    close to the resident size."""
    from transformers import LlamaConfig, LlamaForCausalLM

    from llmquant import QuantConfig, oneshot
    from llmquant.packing import load_packed_model, save_packed_model
    from llmquant.runtime import LlamaKernelRuntime

    torch.manual_seed(0)
    cfg = LlamaConfig(hidden_size=512, intermediate_size=1024, num_hidden_layers=2, num_attention_heads=8,
                      num_key_value_heads=2, head_dim=64, vocab_size=2048, tie_word_embeddings=False,
                      rope_parameters={"rope_type": "default", "rope_theta": 500000.0})
    model = LlamaForCausalLM(cfg).to(torch.bfloat16).cuda().eval()
    oneshot(model, QuantConfig(attn_weight="int8", mlp_weight="int4", head_weight="int8", kv_cache="int8").to_modifier("kernel"))
    path = save_packed_model(model, tmp_path / "m.bin", "local/random-llama", kv_cache_bits=8)
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    before = torch.cuda.memory_allocated()
    loaded = load_packed_model(path, device="cuda", config=cfg)
    peak, resident = torch.cuda.max_memory_allocated() - before, torch.cuda.memory_allocated() - before
    assert peak < resident * 1.25, (peak, resident)
    assert not [n for n, p in loaded.named_parameters() if p.is_meta]
    assert not [n for n, b in loaded.named_buffers() if b is not None and b.is_meta]
    assert loaded.model.layers[0].mlp.down_proj.qdata.dtype == torch.uint8
    for (n1, m1), (n2, m2) in zip(model.named_buffers(), loaded.named_buffers()):
        assert n1 == n2 and torch.equal(m1, m2), n1
    ids = torch.randint(0, 2048, (1, 20), generator=torch.Generator().manual_seed(1)).cuda()
    a = LlamaKernelRuntime(model, 40, 8).generate(ids, 12)
    b = LlamaKernelRuntime(loaded, 40, 8).generate(ids, 12)
    assert torch.equal(a, b)
