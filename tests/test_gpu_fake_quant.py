"""The HIP quantizer against the CPU oracle: bit-exact, on the reference's own case list
(reference tests/test_cuda_kernel.py), through the torch binding and through the bare C ABI."""

import ctypes

import numpy as np
import pytest
import torch

import llmq_oracle as oracle
from conftest import tag_of, to_np

pytestmark = pytest.mark.gpu

DTYPES = [torch.bfloat16, torch.float16, torch.float32]
GROUP = 128


@pytest.fixture(scope="module")
def hip_fake_quantize():
    from llmquant.hip import fake_quantize_hip

    return fake_quantize_hip


def args(bits, strategy="group", group_size=GROUP):
    from llmquant.core.scheme import QuantizationArgs

    if strategy == "group":
        return QuantizationArgs(num_bits=bits, strategy="group", group_size=group_size)
    return QuantizationArgs(num_bits=bits, strategy=strategy)


def same_bits(got: torch.Tensor, want: np.ndarray) -> bool:
    """Equality of values including the sign of zero."""
    got = to_np(got)
    return got.shape == want.shape and np.array_equal(got.view(np.uint32), want.astype(np.float32).view(np.uint32))


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize(
    "shape",
    [(16, GROUP), (2048, 2048), (512, 2048), (2048, 8192), (2, 7, 2048)],
    ids=["single-group", "square", "kv-proj", "down-proj", "activation-3d"],
)
def test_matches_the_oracle_bit_exactly(hip_fake_quantize, bits, dtype, shape):
    torch.manual_seed(0)
    x = (torch.randn(*shape) * 3).to(dtype)
    got, scale = hip_fake_quantize(x.cuda(), args(bits), return_scale=True)
    want = oracle.fake_quantize(to_np(x), bits, tag_of(dtype), "group", GROUP)
    want_scale = oracle.compute_scale(to_np(x), bits, "group", GROUP)[..., 0]
    assert got.dtype == dtype and got.shape == x.shape
    assert same_bits(got, want)
    assert np.array_equal(to_np(scale), want_scale)


@pytest.mark.parametrize("group_size", [32, 128, 256, 2048])
def test_other_group_sizes(hip_fake_quantize, group_size):
    torch.manual_seed(0)
    x = torch.randn(64, 2048).to(torch.bfloat16)
    got = hip_fake_quantize(x.cuda(), args(4, group_size=group_size))
    assert same_bits(got, oracle.fake_quantize(to_np(x), 4, "bf16", "group", group_size))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("group_size", [8, 16, 64, 512, 1024, 4096, 100, 36])
def test_every_kernel_variant(hip_fake_quantize, dtype, group_size):
    """Lane-group widths 1..64 and the block kernel (wide, non power-of-two groups)."""
    torch.manual_seed(1)
    x = (torch.randn(24, group_size * 3) * 2).to(dtype)
    got, scale = hip_fake_quantize(x.cuda(), args(8, group_size=group_size), return_scale=True)
    assert same_bits(got, oracle.fake_quantize(to_np(x), 8, tag_of(dtype), "group", group_size))
    assert np.array_equal(to_np(scale), oracle.compute_scale(to_np(x), 8, "group", group_size)[..., 0])


def test_channel_strategy_is_one_group_per_row(hip_fake_quantize):
    torch.manual_seed(0)
    w = torch.randn(256, 512).to(torch.bfloat16)
    got = hip_fake_quantize(w.cuda(), args(4, strategy="channel"))
    assert same_bits(got, oracle.fake_quantize(to_np(w), 4, "bf16", "channel"))


@pytest.mark.parametrize(
    "name,factory",
    [
        ("all-zero group hits the eps floor", lambda: torch.zeros(4, GROUP)),
        ("tiny values", lambda: torch.full((4, GROUP), 1e-9)),
        ("near-overflow values", lambda: torch.full((4, GROUP), 3e38)),
        ("exact .5 ties round half to even", lambda: torch.arange(512.0).reshape(4, 128) - 256 + 0.5),
    ],
)
def test_edge_cases(hip_fake_quantize, name, factory):
    x = factory()
    got = hip_fake_quantize(x.cuda(), args(8))
    assert same_bits(got, oracle.fake_quantize(to_np(x), 8, "f32", "group", GROUP)), name


def test_non_contiguous_input(hip_fake_quantize):
    torch.manual_seed(0)
    x = torch.randn(GROUP, 64).to(torch.bfloat16).t()
    assert not x.is_contiguous()
    on_device = x.cuda()
    assert not on_device.is_contiguous()
    got = hip_fake_quantize(on_device, args(8))
    assert same_bits(got, oracle.fake_quantize(to_np(x), 8, "bf16", "group", GROUP))


def test_rejects_bad_inputs(hip_fake_quantize):
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        hip_fake_quantize(torch.randn(4, GROUP), args(8))
    with pytest.raises(RuntimeError, match="float32, float16 or bfloat16"):
        hip_fake_quantize(torch.randn(4, GROUP, device="cuda").double(), args(8))


def test_padded_last_axes(hip_fake_quantize):
    torch.manual_seed(0)
    for shape in [(4, 100), (2, 3, 64), (8, 192)]:
        x = torch.randn(*shape).to(torch.bfloat16)
        got = hip_fake_quantize(x.cuda(), args(8))
        assert got.shape == x.shape
        assert same_bits(got, oracle.fake_quantize(to_np(x), 8, "bf16", "group", GROUP)), shape


def test_empty_input(hip_fake_quantize):
    x = torch.empty(0, GROUP, device="cuda", dtype=torch.bfloat16)
    got, scale = hip_fake_quantize(x, args(8), return_scale=True)
    assert got.shape == x.shape and scale.numel() == 0


def test_matches_the_pytorch_form_on_device(hip_fake_quantize):
    """Same answer as the package's own PyTorch statement run on the GPU."""
    from llmquant.core.quant_ops import fake_quantize

    torch.manual_seed(3)
    x = (torch.randn(333, 1024, device="cuda") * 5).to(torch.bfloat16)
    assert torch.equal(hip_fake_quantize(x, args(4)), fake_quantize(x, args(4)))


@pytest.mark.parametrize("bits,pack4", [(8, False), (4, False), (4, True)])
@pytest.mark.parametrize("dtype", DTYPES)
def test_codes_variant(bits, pack4, dtype):
    """quant_group_codes: integer codes and scales, bit-exact; nibble bytes as pack_int4."""
    from llmquant.hip import load_extension

    torch.manual_seed(2)
    x = (torch.randn(37, 1024) * 4).to(dtype)
    codes, scale = load_extension().quant_group_codes(x.cuda(), bits, GROUP, pack4)
    want_codes, want_scale = oracle.quant_group_codes(to_np(x), bits, GROUP)
    if pack4:
        want_codes = oracle.pack_int4(want_codes)
        assert codes.dtype == torch.uint8
    else:
        assert codes.dtype == torch.int8
    assert np.array_equal(codes.cpu().numpy(), want_codes)
    assert np.array_equal(to_np(scale), want_scale)


def test_bare_c_abi_call():
    """The same kernel through ctypes: plain pointers, sizes and a stream, no torch types."""
    from llmquant.hip import load_capi

    lib = load_capi()
    torch.manual_seed(4)
    x = torch.randn(64, 512).to(torch.bfloat16).cuda()
    out = torch.empty_like(x)
    scale = torch.empty(64 * 4, dtype=torch.float32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    rc = lib.llmq_fake_quant_group(x.data_ptr(), out.data_ptr(), scale.data_ptr(), 64 * 4, GROUP, 8,
                                   2, ctypes.c_void_p(stream))
    assert rc == 0, lib.llmq_last_error()
    torch.cuda.synchronize()
    assert same_bits(out, oracle.fake_quantize(to_np(x), 8, "bf16", "group", GROUP))
    rc = lib.llmq_fake_quant_group(x.data_ptr(), out.data_ptr(), None, 4, GROUP, 9, 2, None)
    assert rc == 1 and b"num_bits" in lib.llmq_last_error()
