"""The weight-only GEMM for a few dozen rows (fp16/bf16 activations x int4/int8 weights, no dense
copy of the weight) against the oracle: the float64 closed form  x . (q * s)^T  within the GEMV's
bar (rel-L2 <= 1e-2 for 16-bit outputs, and <= 2e-3 measured against the rounding of the output
alone), the real-mode forward (llmquant/quantizers/real.py:84-91) to the last bit or one output
ulp, ragged sizes, head scales, and agreement with the GEMV kernel row by row."""

import numpy as np
import pytest
import torch

import llmq_oracle as oracle
from conftest import rel_l2, tag_of, to_np

pytestmark = pytest.mark.gpu
GROUP = 128


@pytest.fixture(scope="module")
def ext():
    from llmquant.hip import load_extension

    return load_extension()


def make_case(m, n, k, bits, dtype, out_group=0, seed=0):
    torch.manual_seed(seed)
    w = (torch.randn(n, k) * 0.02).to(torch.bfloat16)
    x = torch.randn(m, k).to(dtype)
    canonical, scales = oracle.canonical_weight(to_np(w), bits, GROUP, None, out_group or None)
    q = torch.from_numpy(oracle.pack_int4(canonical) if bits == 4 else canonical).cuda()
    s = torch.from_numpy(scales).cuda()
    return x, q, s, canonical, scales


def ulp_distance(a, b, dtype):
    """Largest distance, in units of the last place of the 16-bit output type, over the entries of
    ordinary size."""
    if dtype == torch.bfloat16:
        ia = (a.view(np.uint32) >> 16).astype(np.int64)
        ib = (b.view(np.uint32) >> 16).astype(np.int64)
    else:
        ia = a.astype(np.float16).view(np.uint16).astype(np.int64)
        ib = b.astype(np.float16).view(np.uint16).astype(np.int64)
    # sign-magnitude -> monotone integers
    ia = np.where(ia & 0x8000, 0x8000 - ia, ia)
    ib = np.where(ib & 0x8000, 0x8000 - ib, ib)
    # (entries that are small beside the row's typical size are sums that cancel: there the order of
    # the fp32 additions shows in more than the last place, and they are left to the rel-L2 bound)
    big = np.abs(b) > 0.05 * np.sqrt(np.mean(np.square(b.astype(np.float64))))
    return int(np.abs(ia - ib)[big].max())


SPLIT = pytest.mark.parametrize("split", [False, True], ids=["whole rows", "split reduction axis"])


@SPLIT
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,n,k", [(5, 256, 512), (16, 128, 128), (17, 200, 384), (33, 129, 256), (64, 512, 2048),
                                   (70, 96, 640), (1, 16, 128), (48, 64, 1152), (130, 300, 768)])
def test_against_closed_form_and_real_mode(ext, bits, dtype, m, n, k, split):
    x, q, s, canonical, scales = make_case(m, n, k, bits, dtype)
    got = ext.wq_gemm_a16(x.cuda(), q, s, 0, split)
    assert got.shape == (m, n) and got.dtype == dtype
    exact = oracle.gemv_float64(to_np(x), canonical, scales)
    assert rel_l2(to_np(got), exact) <= 2e-3
    # RealQuantLinear's weight-only forward: the same sum, fp32 matmuls per group; the orders of
    # the fp32 additions differ, so equal to within one unit of the output's last place
    want = oracle.real_linear(to_np(x), canonical, scales, tag_of(dtype))
    assert ulp_distance(to_np(got), want, dtype) <= 1
    assert rel_l2(to_np(got), want) <= 2e-3


@SPLIT
@pytest.mark.parametrize("bits", [4, 8])
def test_head_scales(ext, bits, split):
    x, q, s, canonical, scales = make_case(24, 192, 512, bits, torch.bfloat16, out_group=64, seed=1)
    got = ext.wq_gemm_a16(x.cuda(), q, s, 64, split)
    exact = oracle.gemv_float64(to_np(x), canonical, scales, 64)
    assert rel_l2(to_np(got), exact) <= 2e-3


@SPLIT
@pytest.mark.parametrize("bits", [4, 8])
def test_rows_agree_with_the_gemv(ext, bits, split):
    """Each row against the GEMV kernel on that row: two routes to the same sum, one ulp."""
    x, q, s, _, _ = make_case(12, 320, 1024, bits, torch.bfloat16, seed=2)
    got = to_np(ext.wq_gemm_a16(x.cuda(), q, s, 0, split))
    for r0 in range(0, 12, 4):
        rows = to_np(ext.wq_gemv(x[r0:r0 + 4].cuda(), q, s, 0))
        assert ulp_distance(got[r0:r0 + 4], rows, torch.bfloat16) <= 1


@SPLIT
@pytest.mark.parametrize("n,k", [(14336, 4096), (4096, 14336), (8192, 2048), (2048, 8192)])
@pytest.mark.parametrize("m", [8, 64])
def test_llama_shapes_on_sampled_entries(ext, n, k, m, split):
    x, q, s, canonical, scales = make_case(m, n, k, 4, torch.bfloat16, seed=3)
    got = to_np(ext.wq_gemm_a16(x.cuda(), q, s, 0, split))
    rng = np.random.default_rng(0)
    cols = np.sort(rng.choice(n, 64, replace=False))
    exact = oracle.gemv_float64(to_np(x), canonical[cols], scales[cols])
    assert rel_l2(got[:, cols], exact) <= 2e-3


def test_argument_checks(ext):
    x, q, s, _, _ = make_case(8, 64, 256, 4, torch.bfloat16)
    with pytest.raises(RuntimeError, match="float16 or bfloat16"):
        ext.wq_gemm_a16(x.float().cuda(), q, s, 0)
    with pytest.raises(RuntimeError, match="does not match"):
        ext.wq_gemm_a16(x[:, :128].contiguous().cuda(), q, s, 0)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        ext.wq_gemm_a16(x, q, s, 0)
    empty = ext.wq_gemm_a16(x[:0].cuda(), q, s, 0)
    assert empty.shape == (0, 64)


def test_split_form_repeats_itself_and_checks_its_workspace(ext):
    """The slices are added in a fixed order: two runs agree to the bit. The C entry refuses a
    workspace that is too small."""
    import ctypes

    from llmquant.hip import load_capi

    x, q, s, _, _ = make_case(16, 384, 2048, 4, torch.bfloat16, seed=5)
    xd = x.cuda()
    first = ext.wq_gemm_a16(xd, q, s, 0, True)
    for _ in range(3):
        assert torch.equal(ext.wq_gemm_a16(xd, q, s, 0, True), first)
    lib = load_capi()
    need = lib.llmq_wq_gemm_a16_workspace_bytes(16, 384, 16)
    assert need == 4 * 16 * 384 * 4
    assert lib.llmq_wq_gemm_a16_workspace_bytes(16, 384, 4) == 0
    out = torch.empty(16, 384, device="cuda", dtype=torch.bfloat16)
    small = torch.empty(need // 4 - 4, device="cuda", dtype=torch.float32)
    rc = lib.llmq_wq_gemm_a16_split(xd.data_ptr(), q.data_ptr(), s.data_ptr(), out.data_ptr(), small.data_ptr(),
                                    small.numel() * 4, 16, 384, 16, 128, 0, 4, 2, None)
    assert rc != 0 and b"workspace" in lib.llmq_last_error()
