"""Property tests (hypothesis) of the quantizer's host functions and the oracle, on the CPU: the
invariants the reference's tests state on fixed inputs (tests/test_quantization.py,
tests/test_grouping.py, tests/test_packing.py, tests/test_moe.py), over generated ones."""

import numpy as np
import torch
from hypothesis import given, settings, strategies as st

import llmq_oracle as oracle
from llmquant.core import observers as obs
from llmquant.core.quant_ops import fake_quantize, quantize
from llmquant.core.scheme import QuantizationArgs
from llmquant.packing.format import read_packed, write_packed
from llmquant.packing.packing import pack_int4, unpack_int4
from llmquant.quantizers import route_plan

FAST = settings(max_examples=40, deadline=None)
seeds = st.integers(0, 2 ** 31 - 1)
bits = st.sampled_from([4, 8])


def tensor(seed, *shape, scale=1.0):
    gen = torch.Generator().manual_seed(seed)
    # a wide dynamic range: exponents spread over +-8 octaves
    return torch.randn(*shape, generator=gen) * scale * torch.exp2(torch.randint(-8, 9, shape, generator=gen).float())


@FAST
@given(seeds, bits, st.integers(1, 5), st.sampled_from([32, 64, 128]))
def test_torch_fake_quantize_is_the_oracle_bit_for_bit(seed, num_bits, rows, gs):
    x = tensor(seed, rows, 3 * gs)
    args = QuantizationArgs(num_bits=num_bits, strategy="group", group_size=gs)
    got = fake_quantize(x, args)
    want = oracle.fake_quantize(x.numpy(), num_bits, "f32", "group", gs)
    assert np.array_equal(got.numpy(), want)
    got16 = fake_quantize(x.to(torch.bfloat16), args)
    want16 = oracle.fake_quantize(x.to(torch.bfloat16).float().numpy(), num_bits, "bf16", "group", gs)
    assert np.array_equal(got16.float().numpy(), want16)


@FAST
@given(seeds, bits, st.sampled_from([24, 64, 100]))
def test_padding_is_numerically_free(seed, num_bits, width):
    """A last axis shorter than the group quantizes as a group of its own width: the zeros added to
    fill the group change neither the abs-max nor any code."""
    x = tensor(seed, 4, width)
    padded = fake_quantize(x, QuantizationArgs(num_bits=num_bits, strategy="group", group_size=128))
    exact = fake_quantize(x, QuantizationArgs(num_bits=num_bits, strategy="group", group_size=width))
    assert torch.equal(padded, exact)


@FAST
@given(seeds, bits, st.sampled_from([64, 128, 384]))
def test_channel_is_one_group_over_the_whole_row(seed, num_bits, k):
    x = tensor(seed, 3, k)
    per_channel = fake_quantize(x, QuantizationArgs(num_bits=num_bits, strategy="channel"))
    one_group = fake_quantize(x, QuantizationArgs(num_bits=num_bits, strategy="group", group_size=k))
    assert torch.equal(per_channel, one_group)


@FAST
@given(seeds, bits)
def test_codes_survive_a_second_quantization(seed, num_bits):
    """Quantizing the dequantized values gives the same codes again (the scale may move by an ulp)."""
    x = tensor(seed, 6, 256)
    args = QuantizationArgs(num_bits=num_bits, strategy="group", group_size=128)
    scale = obs.compute_scale(x, args)
    codes = quantize(obs.group_view(x, 128), scale, args)
    again_in = (codes * scale).reshape(6, 256)
    scale2 = obs.compute_scale(again_in, args)
    codes2 = quantize(obs.group_view(again_in, 128), scale2, args)
    assert torch.equal(codes, codes2)
    assert torch.allclose(scale, scale2, rtol=3e-7, atol=0)
    qmax = 2 ** (num_bits - 1) - 1
    assert codes.abs().amax(dim=-1).eq(qmax).all()  # the abs-max element lands on +-qmax


@FAST
@given(seeds, bits, st.integers(0, 5))
def test_rows_and_groups_are_quantized_independently(seed, num_bits, victim):
    x = tensor(seed, 6, 256)
    args = QuantizationArgs(num_bits=num_bits, strategy="group", group_size=128)
    base = fake_quantize(x, args)
    y = x.clone()
    y[victim, :128] *= 37.0
    moved = fake_quantize(y, args)
    keep = torch.ones(6, 256, dtype=torch.bool)
    keep[victim, :128] = False
    assert torch.equal(base[keep], moved[keep])


@FAST
@given(seeds, st.sampled_from([(4, 100, None), (3, 256, 64), (2, 192, 64), (5, 128, None), (2, 96, 32)]))
def test_group_view_and_ungroup_are_inverse(seed, case):
    rows, k, head_dim = case
    x = tensor(seed, rows, k)
    grouped = obs.group_view(x, 128, head_dim)
    assert grouped.shape[-1] == 128
    assert torch.equal(obs.ungroup(grouped, x.shape, 128, head_dim), x)
    want = oracle.group_view(x.numpy(), 128, head_dim)
    assert np.array_equal(grouped.numpy(), want)


@FAST
@given(seeds, st.integers(1, 6), st.sampled_from([2, 8, 64, 128]))
def test_nibble_packing_is_a_bijection(seed, rows, width):
    gen = torch.Generator().manual_seed(seed)
    codes = torch.randint(-8, 8, (rows, width), generator=gen, dtype=torch.int8)
    packed = pack_int4(codes)
    assert packed.dtype == torch.uint8 and packed.shape == (rows, width // 2)
    assert torch.equal(unpack_int4(packed), codes)
    assert np.array_equal(packed.numpy(), oracle.pack_int4(codes.numpy()))
    # and the other way: every byte value is the image of exactly one pair of codes
    every = torch.arange(256, dtype=torch.uint8).reshape(1, 256)
    assert torch.equal(pack_int4(unpack_int4(every)), every)


@FAST
@given(seeds, st.integers(1, 4))
def test_packed_file_round_trip(tmp_path_factory, seed, count):
    gen = torch.Generator().manual_seed(seed)
    dtypes = [torch.uint8, torch.int8, torch.float32, torch.bfloat16]
    tensors = {}
    for i in range(count):
        shape = tuple(int(v) for v in torch.randint(1, 9, (int(torch.randint(1, 4, (1,), generator=gen)),), generator=gen))
        dt = dtypes[int(torch.randint(0, 4, (1,), generator=gen))]
        raw = torch.randn(*shape, generator=gen) * 50
        tensors[f"layer.{i}.t"] = raw.to(dt) if dt.is_floating_point else raw.clamp(-100, 100).to(torch.int16).to(dt)
    path = tmp_path_factory.mktemp("packed") / "w.llmq"
    write_packed(path, tensors, {"seed": seed})
    back, meta = read_packed(path)
    assert meta == {"seed": seed} and list(back) == list(tensors)
    for name, t in tensors.items():
        assert back[name].dtype == t.dtype and torch.equal(back[name], t)
    names = {torch.uint8: "uint8", torch.int8: "int8", torch.float32: "float32", torch.bfloat16: "bfloat16"}
    as_np = {k: (names[v.dtype], v.view(torch.uint16).numpy() if v.dtype == torch.bfloat16 else v.numpy())
             for k, v in tensors.items()}
    assert path.read_bytes() == oracle.packed_file_bytes(as_np, {"seed": seed})  # the bytes, not just the values


@FAST
@given(seeds, st.integers(1, 9), st.sampled_from([(4, 2), (8, 4), (64, 8), (3, 3)]), st.sampled_from([2, 4, 8]))
def test_route_plan_invariants(seed, tokens, shape, limit):
    experts, top_k = shape
    gen = torch.Generator().manual_seed(seed)
    index = torch.stack([torch.randperm(experts, generator=gen)[:top_k] for _ in range(tokens)])
    order, (block_expert, block_row0, block_rows) = route_plan(index, experts, limit)
    expert_of_row = index.reshape(-1)[order]
    assert (expert_of_row[1:] >= expert_of_row[:-1]).all()  # sorted by expert, stably
    covered = torch.zeros(index.numel(), dtype=torch.int32)
    for e, r0, n in zip(block_expert.tolist(), block_row0.tolist(), block_rows.tolist()):
        assert 0 <= n <= limit
        if n:
            assert (expert_of_row[r0:r0 + n] == e).all()
            covered[r0:r0 + n] += 1
    assert (covered == 1).all()
