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


# ---- the tiled form for prompt-sized M ---------------------------------------------------------------------


#: The tiled GEMM has two tile shapes with the same arithmetic: 128 x 256 (eight waves) and 64 x 128 (four waves,
#: for outputs of few wide tiles). LLMQ_A16_TILE pins one whatever the problem; None is the library's own choice.
SHAPES = pytest.mark.parametrize("tile", ["wide", "narrow", None], ids=["128x256", "64x128", "own choice"])


@pytest.fixture(autouse=True)
def no_tile_shape_left_pinned():
    import os

    yield
    os.environ.pop("LLMQ_A16_TILE", None)


def tile_case(ext, m, n, k, bits, out_group=0, head_dim=None, seed=0, scale=1.0, offset=0.0, tile=None,
              dtype=torch.bfloat16):
    """x [m, k] bf16 (or fp16) against a quantized [n, k] weight through wq_gemm_a16_tile; returns the result and
    the oracle's operands (activation padded the way the weight was)."""
    import os

    if tile is None:
        os.environ.pop("LLMQ_A16_TILE", None)
    else:
        os.environ["LLMQ_A16_TILE"] = tile
    torch.manual_seed(seed)
    w = (torch.randn(n, k) * 0.02).to(dtype)
    x = (torch.randn(m, k) * scale + offset).to(dtype)
    canonical, scales = oracle.canonical_weight(to_np(w), bits, GROUP, head_dim, out_group or None)
    q = torch.from_numpy(oracle.pack_int4(canonical) if bits == 4 else canonical).cuda()
    s = torch.from_numpy(scales).cuda()
    padded = oracle.pad_activation(to_np(x), GROUP, head_dim)
    got = ext.wq_gemm_a16_tile(torch.from_numpy(padded).to(dtype).cuda(), q, s, out_group)
    return got, padded, canonical, scales


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("m,n,k", [(128, 256, 128), (65, 256, 256), (130, 300, 768), (512, 512, 2048), (300, 70, 384),
                                   (129, 257, 1152), (1, 16, 128), (256, 1024, 8192), (65, 70, 1024),
                                   (1023, 66, 2048)])
@SHAPES
def test_tiled_gemm_against_the_oracle(ext, bits, m, n, k, tile):
    """Whole outputs against the float64 closed form and the real-mode forward: full tiles, ragged M and N
    (rows and columns past the end are clamped for the loads and dropped at the store), one group, rows long
    enough that the reduction axis is split across workgroups, and split outputs whose element count is not a
    multiple of four (the slice addition then walks its values one at a time)."""
    got, x, canonical, scales = tile_case(ext, m, n, k, bits, seed=m + n, tile=tile)
    assert got.shape == (m, n) and got.dtype == torch.bfloat16
    exact = oracle.gemv_float64(x, canonical, scales)
    assert rel_l2(to_np(got), exact) <= 2e-3
    real = oracle.real_linear(x, canonical, scales, "bf16")
    assert ulp_distance(to_np(got), real, torch.bfloat16) <= 1
    assert (to_np(got) == real).mean() > 0.99


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("m,n,k", [(128, 256, 128), (130, 300, 768), (512, 512, 2048), (300, 70, 384), (256, 1024, 8192),
                                   (65, 70, 1024), (512, 3072, 2048)])
@SHAPES
def test_tiled_gemm_float16_against_the_oracle(ext, bits, m, n, k, tile):
    """float16 activations: the codes enter the matrix core as themselves (the bias of the bf16 form is taken off
    the operand, exactly), so there is no correction term; same bars as the bf16 form, with float16's rounding of
    the output. A second case with activations near float16's largest values: products and sums are fp32, nothing
    overflows on the way."""
    got, x, canonical, scales = tile_case(ext, m, n, k, bits, seed=m + n, tile=tile, dtype=torch.float16)
    assert got.shape == (m, n) and got.dtype == torch.float16
    exact = oracle.gemv_float64(x, canonical, scales)
    assert rel_l2(to_np(got), exact) <= 3e-4
    real = oracle.real_linear(x, canonical, scales, "f16")
    assert ulp_distance(to_np(got), real, torch.float16) <= 1
    assert (to_np(got) == real).mean() > 0.99
    if (m, n, k) == (512, 512, 2048):
        # one scale row per 64 weight rows, and heads of 64 padded to groups
        for spec in (dict(out_group=64), dict(head_dim=64)):
            got, x, canonical, scales = tile_case(ext, m, n, k, bits, seed=4, tile=tile, dtype=torch.float16, **spec)
            og = spec.get("out_group")
            full = np.repeat(scales, og, axis=0)[:n] if og else scales
            assert rel_l2(to_np(got), oracle.gemv_float64(x, canonical, full)) <= 3e-4
    if (m, n, k) == (130, 300, 768):
        got, x, canonical, scales = tile_case(ext, m, n, k, bits, seed=2, tile=tile, dtype=torch.float16, scale=2000.0,
                                              offset=30000.0)
        assert np.abs(x).max() > 30000 and torch.isfinite(got).all()
        assert rel_l2(to_np(got), oracle.gemv_float64(x, canonical, scales)) <= 3e-4


@pytest.mark.parametrize("bits", [4, 8])
def test_gate_up_silu_epilogue_float16(ext, bits):
    """The two-launch MLP on float16 activations against the three launches, equal to the bit (wide tile pinned, as
    for bf16), and the norm in front of it written as prepared rows."""
    import os

    os.environ["LLMQ_A16_TILE"] = "wide"
    m, inter, k, n_down = 200, 256, 256, 300
    x, q_gu, s_gu, q_d, s_d, _ = mlp_case(m, inter, k, n_down, bits, seed=9)
    x = (x.float() * 0.5).half()
    gate_up = ext.wq_gemm_a16_tile(x, q_gu, s_gu, 0)
    act = ext.silu_mul(gate_up[:, :inter], gate_up[:, inter:])
    want = ext.wq_gemm_a16_tile(act, q_d, s_d, 0)
    workspace = ext.wq_gemm_a16_tile_gate_up_silu(x, q_gu, s_gu, 0, n_down)
    got = ext.wq_gemm_a16_tile_prepared(workspace, m, q_d, s_d, 0, torch.float16)
    assert got.dtype == torch.float16 and torch.equal(got, want)
    weight = (1 + 0.1 * torch.randn(k, device="cuda")).half()
    delta = torch.randn_like(x)
    hidden, normed = ext.add_rmsnorm(x, delta, weight, 1e-5)
    want = ext.wq_gemm_a16_tile_prepared(ext.wq_gemm_a16_tile_gate_up_silu(normed, q_gu, s_gu, 0, n_down), m, q_d, s_d, 0,
                                         torch.float16)
    got_hidden, ws = ext.add_rmsnorm_prepared(x, delta, weight, 1e-5, max(2 * inter, n_down))
    got = ext.wq_gemm_a16_tile_prepared(ext.wq_gemm_a16_tile_gate_up_silu_prepared(ws, m, q_gu, s_gu, 0, n_down, torch.float16),
                                        m, q_d, s_d, 0, torch.float16)
    assert torch.equal(got_hidden, hidden) and torch.equal(got, want)


@pytest.mark.parametrize("bits", [4, 8])
def test_tiled_gemm_with_one_signed_activation(ext, bits):
    """Activations that do not cancel (all positive, mean 3): the codes enter the matrix core with an offset
    (code + 24 or + 128) that is taken out per group through the activation's sum, and this is the input on
    which that term is largest beside the result."""
    got, x, canonical, scales = tile_case(ext, 256, 512, 1024, bits, seed=5, scale=0.5, offset=3.0)
    exact = oracle.gemv_float64(x, canonical, scales)
    assert rel_l2(to_np(got), exact) <= 2e-3
    wide = ext.wq_gemm_a16_tile((torch.from_numpy(x) * 0 + 1).to(torch.bfloat16).cuda(),
                                torch.from_numpy(oracle.pack_int4(canonical) if bits == 4 else canonical).cuda(),
                                torch.from_numpy(scales).cuda(), 0)
    ones = oracle.gemv_float64(np.ones_like(x), canonical, scales)   # x = 1: the plain row sums of the weight
    assert rel_l2(to_np(wide), ones) <= 4e-3


PREFILL_SHAPES = {
    "q|k|v 3072x2048 int8, one scale row per head": dict(n=3072, k=2048, bits=8, out_group=64),
    "o_proj 2048x2048 int8, heads of 64 padded to groups": dict(n=2048, k=2048, bits=8, head_dim=64),
    "gate|up 16384x2048 int4": dict(n=16384, k=2048, bits=4),
    "down 2048x8192 int4": dict(n=2048, k=8192, bits=4),
}


@SHAPES
@pytest.mark.parametrize("name", list(PREFILL_SHAPES))
def test_tiled_gemm_at_the_prompt_pass_shapes(ext, name, tile):
    """The four projections of a 512-token prompt pass of the Llama-3.2-1B configuration, on 96 x 128 sampled
    outputs (and the last rows and columns) against the float64 closed form, rel-L2 <= 2e-3, and against the
    real-mode forward restricted to the sample."""
    spec = dict(PREFILL_SHAPES[name])
    m, n, k, bits = 512, spec.pop("n"), spec.pop("k"), spec.pop("bits")
    got, x, canonical, scales = tile_case(ext, m, n, k, bits, seed=11, tile=tile, **spec)
    out_group = spec.get("out_group")
    rng = np.random.default_rng(3)
    rows = np.unique(np.concatenate([rng.choice(m, 96, replace=False), [m - 1]]))
    cols = np.unique(np.concatenate([rng.choice(n, 128, replace=False), [n - 1]]))
    full_scales = np.repeat(scales, out_group, axis=0)[:n] if out_group else scales
    exact = oracle.gemv_float64(x[rows], canonical[cols], full_scales[cols])
    sample = to_np(got)[np.ix_(rows, cols)]
    assert rel_l2(sample, exact) <= 2e-3
    real = oracle.real_linear(x[rows], canonical[cols], full_scales[cols], "bf16")
    assert (sample == real).mean() > 0.99 and ulp_distance(sample, real, torch.bfloat16) <= 1


@pytest.mark.parametrize("n,k", [(14336, 4096), (4096, 14336)])
@pytest.mark.parametrize("m", [128, 2048])
def test_tiled_gemm_at_llama_8b_mlp_shapes(ext, n, k, m):
    got, x, canonical, scales = tile_case(ext, m, n, k, 4, seed=13)
    rng = np.random.default_rng(4)
    rows = np.sort(rng.choice(m, 64, replace=False))
    cols = np.sort(rng.choice(n, 96, replace=False))
    exact = oracle.gemv_float64(x[rows], canonical[cols], scales[cols])
    assert rel_l2(to_np(got)[np.ix_(rows, cols)], exact) <= 2e-3


def test_tiled_gemm_argument_checks(ext):
    x, q, s, _, _ = make_case(128, 256, 256, 4, torch.bfloat16)
    assert ext.wq_gemm_a16_tile(x.cuda(), q, s, 0).shape == (128, 256)
    with pytest.raises(RuntimeError, match="bfloat16 or float16"):
        ext.wq_gemm_a16_tile(x.cuda().float(), q, s, 0)
    with pytest.raises(RuntimeError, match="does not match qweight"):
        ext.wq_gemm_a16_tile(x.cuda()[:, :128].contiguous(), q, s, 0)
    with pytest.raises(RuntimeError, match="wscale must be"):
        ext.wq_gemm_a16_tile(x.cuda(), q, s[:-1], 0)
    assert ext.wq_gemm_a16_tile(x.cuda()[:0], q, s, 0).shape == (0, 256)


@pytest.mark.parametrize("bits,layout", [(4, {}), (8, {"out_group": 64}), (4, {"head_dim": 64})])
def test_module_takes_the_tiled_gemm_for_a_prompt(ext, bits, layout):
    """KernelQuantLinear on a prompt-sized bf16 batch against a wide weight: the tiled fused GEMM runs (the
    dense branch is made to fail loudly), padded heads and head scales included, and the result is the
    real-mode sum."""
    import torch.nn as nn

    from llmquant.core.scheme import QuantizationArgs, QuantizationScheme
    from llmquant.quantizers import KernelQuantLinear
    from llmquant.quantizers.kernel import tiled_gemm_pays

    torch.manual_seed(21)
    linear = nn.Linear(1024, 8192, bias=False).to(torch.bfloat16).cuda()
    scheme = QuantizationScheme(weights=QuantizationArgs(num_bits=bits, strategy="group", group_size=GROUP, **layout),
                                input_activations=None)
    module = KernelQuantLinear.from_linear(linear, scheme)
    module._dequantized_weight = module._dense = None
    m = 200
    assert tiled_gemm_pays(m, 8192, module.qdata.shape[1]) and not tiled_gemm_pays(2048, 8192, 8)
    x = torch.randn(2, m // 2, 1024).to(torch.bfloat16)
    got = module(x.cuda())
    assert got.shape == (2, m // 2, 8192) and got.dtype == torch.bfloat16
    canonical, scales = oracle.canonical_weight(to_np(linear.weight), bits, GROUP, layout.get("head_dim"),
                                                layout.get("out_group"))
    padded = oracle.pad_activation(to_np(x).reshape(m, -1), GROUP, layout.get("head_dim"))
    rng = np.random.default_rng(5)
    cols = np.sort(rng.choice(8192, 256, replace=False))
    og = layout.get("out_group")
    full_scales = np.repeat(scales, og, axis=0)[:8192] if og else scales
    exact = oracle.gemv_float64(padded, canonical[cols], full_scales[cols])
    assert rel_l2(to_np(got).reshape(m, -1)[:, cols], exact) <= 2e-3


@pytest.mark.parametrize("bits,layout", [(8, {"out_group": 64}), (4, {})])
def test_module_keeps_the_fused_gemm_for_100_rows_of_a_narrow_weight(ext, bits, layout):
    """KernelQuantLinear on 100 rows against a q|k|v-sized weight (3072 x 2048): two launches of the fused GEMM for a
    few dozen rows run (the dense branch and the tiled GEMM are made to fail loudly), and the result is the
    real-mode sum; with heads padded to groups the dense branch on the real width keeps such a batch."""
    import torch.nn as nn

    from llmquant.core.scheme import QuantizationArgs, QuantizationScheme
    from llmquant.quantizers import KernelQuantLinear

    torch.manual_seed(22)
    linear = nn.Linear(2048, 3072, bias=False).to(torch.bfloat16).cuda()
    scheme = QuantizationScheme(weights=QuantizationArgs(num_bits=bits, strategy="group", group_size=GROUP, **layout),
                                input_activations=None)
    module = KernelQuantLinear.from_linear(linear, scheme)
    module._dequantized_weight = module._dense = None
    m = 100
    x = torch.randn(m, 2048).to(torch.bfloat16)
    real_tile = module._ext.wq_gemm_a16_tile
    try:
        module._ext.wq_gemm_a16_tile = None
        got = module(x.cuda())
    finally:
        module._ext.wq_gemm_a16_tile = real_tile
    assert got.shape == (m, 3072) and got.dtype == torch.bfloat16
    canonical, scales = oracle.canonical_weight(to_np(linear.weight), bits, GROUP, None, layout.get("out_group"))
    og = layout.get("out_group")
    full_scales = np.repeat(scales, og, axis=0)[:3072] if og else scales
    exact = oracle.gemv_float64(to_np(x), canonical, full_scales)
    assert rel_l2(to_np(got), exact) <= 2e-3
    assert torch.equal(got[:64], module(x[:64].cuda())) and torch.equal(got[64:], module(x[64:].cuda()))
    padded = KernelQuantLinear.from_linear(nn.Linear(2048, 2048, bias=False).to(torch.bfloat16).cuda(), QuantizationScheme(
        weights=QuantizationArgs(num_bits=8, strategy="group", group_size=GROUP, head_dim=64), input_activations=None))
    calls = []
    dense = padded._dense
    padded._dense = lambda rows, real_width=False: (calls.append(real_width), dense(rows, real_width))[1]
    padded(torch.randn(m, 2048).to(torch.bfloat16).cuda())
    assert calls == [True]


# ---- gate|up with silu(gate) * up written as down_proj's prepared activation ------------------------------------


def mlp_case(m, inter, k, n_down, bits, seed, out_group=0):
    torch.manual_seed(seed)
    x = torch.randn(m, k).to(torch.bfloat16)
    w_gu = (torch.randn(2 * inter, k) * 0.05).to(torch.bfloat16)
    w_d = (torch.randn(n_down, inter) * 0.05).to(torch.bfloat16)
    c_gu, s_gu = oracle.canonical_weight(to_np(w_gu), bits, GROUP, None, out_group or None)
    c_d, s_d = oracle.canonical_weight(to_np(w_d), bits, GROUP, None, None)
    pack = (lambda c: oracle.pack_int4(c)) if bits == 4 else (lambda c: c)
    return (x.cuda(), torch.from_numpy(pack(c_gu)).cuda(), torch.from_numpy(s_gu).cuda(),
            torch.from_numpy(pack(c_d)).cuda(), torch.from_numpy(s_d).cuda(), (to_np(x), c_gu, s_gu, c_d, s_d))


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("m,inter,k,n_down,out_group", [
    (512, 1024, 384, 768, 0),   # whole tiles
    (200, 256, 256, 300, 0),    # ragged rows, ragged down_proj columns
    (65, 128, 128, 64, 0),      # one tile, one group
    (130, 384, 512, 2048, 64),  # gate|up scales in tiles of 64 rows
])
def test_gate_up_silu_epilogue_gives_the_bits_of_the_three_launches(ext, bits, m, inter, k, n_down, out_group):
    """llmq_wq_gemm_a16_tile_gate_up_silu + llmq_wq_gemm_a16_tile_prepared against llmq_wq_gemm_a16_tile ->
    llmq_silu_mul -> llmq_wq_gemm_a16_tile on the same operands: equal to the bit. (Reduction axes of at most
    seven groups here: there the plain tiled GEMM does not split the axis either, so its fp32 sums run in the
    order of the fused launch's. The rounding points are the same in any case; the longer axis is below. The
    128 x 256 tile is pinned for the three launches: the epilogue is laid out for it, and the 64 x 128 tile adds
    the two halves of every group separately.)"""
    import os

    os.environ["LLMQ_A16_TILE"] = "wide"
    x, q_gu, s_gu, q_d, s_d, _ = mlp_case(m, inter, k, n_down, bits, seed=m + inter, out_group=out_group)
    gate_up = ext.wq_gemm_a16_tile(x, q_gu, s_gu, out_group)
    act = ext.silu_mul(gate_up[:, :inter], gate_up[:, inter:])
    want = ext.wq_gemm_a16_tile(act, q_d, s_d, 0)
    workspace = ext.wq_gemm_a16_tile_gate_up_silu(x, q_gu, s_gu, out_group, n_down)
    got = ext.wq_gemm_a16_tile_prepared(workspace, m, q_d, s_d, 0)
    assert got.shape == want.shape == (m, n_down) and got.dtype == torch.bfloat16
    assert torch.equal(got, want)
    # and the transformers form of the same thing on the same bf16 tensors
    act_hf = torch.nn.functional.silu(gate_up[:, :inter]) * gate_up[:, inter:]
    assert torch.equal(act, act_hf)


@pytest.mark.parametrize("bits", [4, 8])
def test_gate_up_silu_epilogue_against_float64_on_a_long_axis(ext, bits):
    """The Llama-3.2-1B MLP's reduction axes (2048 into gate|up, a cut of the 8192 into down_proj) against the
    whole MLP in float64 on the quantized weights, with the bf16 roundings of the two Linear outputs and of the
    activation applied where the modules apply them: rel-L2 <= 3e-3 (two chained bf16 results)."""
    m, inter, k, n_down = 256, 2048, 2048, 512
    x, q_gu, s_gu, q_d, s_d, (xn, c_gu, sc_gu, c_d, sc_d) = mlp_case(m, inter, k, n_down, bits, seed=3)
    workspace = ext.wq_gemm_a16_tile_gate_up_silu(x, q_gu, s_gu, 0, n_down)
    got = ext.wq_gemm_a16_tile_prepared(workspace, m, q_d, s_d, 0)
    bf = lambda a: torch.from_numpy(np.asarray(a, dtype=np.float32)).to(torch.bfloat16).float().numpy().astype(np.float64)
    gu = bf(oracle.gemv_float64(xn, c_gu, sc_gu))
    g, u = gu[:, :inter], gu[:, inter:]
    act = bf(bf(g / (1.0 + np.exp(-g))) * u)
    want = oracle.gemv_float64(act.astype(np.float32), c_d, sc_d)
    assert rel_l2(to_np(got), want) <= 3e-3
    # the three launches on the same operands: the same roundings, sums possibly in another order
    gate_up = ext.wq_gemm_a16_tile(x, q_gu, s_gu, 0)
    unfused = ext.wq_gemm_a16_tile(ext.silu_mul(gate_up[:, :inter], gate_up[:, inter:]), q_d, s_d, 0)
    assert rel_l2(to_np(got), to_np(unfused).astype(np.float64)) <= 2e-3


def test_gate_up_silu_epilogue_argument_checks(ext):
    x, q_gu, s_gu, q_d, s_d, _ = mlp_case(128, 128, 128, 64, 4, seed=1)
    with pytest.raises(RuntimeError, match="multiple of 128"):
        ext.wq_gemm_a16_tile_gate_up_silu(x, q_gu[:192], s_gu[:192], 0, 64)
    with pytest.raises(RuntimeError, match="bfloat16 or float16"):
        ext.wq_gemm_a16_tile_gate_up_silu(x.float(), q_gu, s_gu, 0, 64)
    workspace = ext.wq_gemm_a16_tile_gate_up_silu(x, q_gu, s_gu, 0, 64)
    with pytest.raises(RuntimeError, match="this GEMM needs"):
        ext.wq_gemm_a16_tile_prepared(workspace[:16], 128, q_d, s_d, 0)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("with_delta", [False, True], ids=["norm", "add+norm"])
@pytest.mark.parametrize("m,k,n", [(512, 2048, 3072), (200, 384, 520), (65, 128, 64), (130, 4096, 1024)])
def test_rmsnorm_into_prepared_form_gives_the_bits_of_norm_then_gemm(ext, m, k, n, with_delta, bits):
    """llmq_add_rmsnorm_prepared + llmq_wq_gemm_a16_tile_prepared against llmq_add_rmsnorm -> llmq_wq_gemm_a16_tile:
    the residual sum, the prepared chunks (eight consecutive normed values in the order 0, 4, 1, 5, 2, 6, 3, 7) and
    the GEMM's output equal to the bit; the norm itself against the oracle's LlamaRMSNorm (the mean of squares is
    summed in another order on the GPU: a last-place difference in 1 / rms moves a few results by one bf16 step)."""
    torch.manual_seed(m + k)
    x = (torch.randn(m, k, device="cuda") * 1.5).to(torch.bfloat16)
    delta = torch.randn(m, k, device="cuda").to(torch.bfloat16) if with_delta else None
    weight = (1 + 0.1 * torch.randn(k, device="cuda")).to(torch.bfloat16)
    width = GROUP if bits == 8 else GROUP // 2
    q = torch.randint(0, 256, (n, k // GROUP, width), dtype=torch.uint8, device="cuda")
    q = q.view(torch.int8) if bits == 8 else q
    sw = torch.rand(n, k // GROUP, device="cuda") * 0.004 + 0.001
    if with_delta:
        want_sum, normed = ext.add_rmsnorm(x, delta, weight, 1e-5)
    else:
        want_sum, normed = x, ext.rmsnorm(x, weight, 1e-5)
    want = ext.wq_gemm_a16_tile(normed, q, sw, 0)
    got_sum, workspace = ext.add_rmsnorm_prepared(x, delta, weight, 1e-5, n)
    prepared = workspace.view(torch.uint8)[: m * k * 2].clone()
    got = ext.wq_gemm_a16_tile_prepared(workspace, m, q, sw, 0)
    assert torch.equal(got_sum, want_sum) and torch.equal(got, want)
    chunks = normed.view(m, k // 8, 8)[:, :, [0, 4, 1, 5, 2, 6, 3, 7]].contiguous()
    assert torch.equal(prepared, chunks.view(torch.uint8).flatten())
    summed = to_np(x).astype(np.float32) + (to_np(delta).astype(np.float32) if with_delta else 0)
    summed = oracle.round_to(summed, "bf16") if with_delta else summed
    want_normed = oracle.llama_rmsnorm(summed, to_np(weight), 1e-5, "bf16")
    assert (to_np(normed) == want_normed).mean() > 0.99 and rel_l2(to_np(normed), want_normed) <= 1e-3


@pytest.mark.parametrize("bits", [4, 8])
def test_gate_up_silu_epilogue_on_prepared_rows(ext, bits):
    """The gated MLP of a prompt from the norm on: add_rmsnorm_prepared -> gate_up_silu_prepared -> prepared against
    add_rmsnorm -> gate_up_silu -> prepared, equal to the bit."""
    m, inter, k, n_down = 300, 2560, 512, 640
    x, q_gu, s_gu, q_d, s_d, _ = mlp_case(m, inter, k, n_down, bits, seed=5)
    delta = torch.randn_like(x)
    weight = (1 + 0.1 * torch.randn(k, device="cuda")).to(torch.bfloat16)
    hidden, normed = ext.add_rmsnorm(x, delta, weight, 1e-6)
    want = ext.wq_gemm_a16_tile_prepared(ext.wq_gemm_a16_tile_gate_up_silu(normed, q_gu, s_gu, 0, n_down), m, q_d, s_d, 0)
    got_hidden, workspace = ext.add_rmsnorm_prepared(x, delta, weight, 1e-6, max(2 * inter, n_down))
    down_ws = ext.wq_gemm_a16_tile_gate_up_silu_prepared(workspace, m, q_gu, s_gu, 0, n_down)
    got = ext.wq_gemm_a16_tile_prepared(down_ws, m, q_d, s_d, 0)
    assert torch.equal(got_hidden, hidden) and torch.equal(got, want)
    assert float(want.float().abs().mean()) > 0


def test_rmsnorm_into_prepared_form_argument_checks(ext):
    x = torch.randn(64, 256, device="cuda").to(torch.bfloat16)
    weight = torch.ones(256, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="bfloat16 or float16"):
        ext.add_rmsnorm_prepared(x.float(), None, weight.float(), 1e-5, 128)
    with pytest.raises(RuntimeError, match="multiple of 128"):
        ext.add_rmsnorm_prepared(x[:, :200].contiguous(), None, weight[:200].contiguous(), 1e-5, 128)
    with pytest.raises(RuntimeError, match="must match"):
        ext.add_rmsnorm_prepared(x, x[:32], weight, 1e-5, 128)
    _, workspace = ext.add_rmsnorm_prepared(x, None, weight, 1e-5, 128)
    q = torch.randint(0, 256, (512, 2, 64), dtype=torch.uint8, device="cuda")
    with pytest.raises(RuntimeError, match="this GEMM needs"):
        ext.wq_gemm_a16_tile_gate_up_silu_prepared(workspace[:16], 64, q, torch.ones(512, 2, device="cuda"), 0, 64)


def test_gate_up_silu_epilogue_at_the_llama_1b_prompt_shape(ext):
    """The MLP of a 512-token prompt of the Llama-3.2-1B configuration (2048 -> 2 x 8192 -> 2048, int4): 4 x 64
    tiles, the shape the runtime takes this path on. Bit-equal to the three launches (the plain gate|up GEMM has
    256 tiles and keeps its reduction axis whole too; down_proj's plan is the same in both), and the prepared
    activation the epilogue leaves is, byte for byte, what the preparation pass makes of silu(gate) * up."""
    m, inter, k, n_down = 512, 8192, 2048, 2048
    torch.manual_seed(11)
    x = torch.randn(m, k, device="cuda").to(torch.bfloat16)
    q_gu = torch.randint(0, 256, (2 * inter, k // GROUP, GROUP // 2), dtype=torch.uint8, device="cuda")
    s_gu = torch.rand(2 * inter, k // GROUP, device="cuda") * 0.004 + 0.001
    q_d = torch.randint(0, 256, (n_down, inter // GROUP, GROUP // 2), dtype=torch.uint8, device="cuda")
    s_d = torch.rand(n_down, inter // GROUP, device="cuda") * 0.004 + 0.001
    gate_up = ext.wq_gemm_a16_tile(x, q_gu, s_gu, 0)
    act = ext.silu_mul(gate_up[:, :inter], gate_up[:, inter:])
    want = ext.wq_gemm_a16_tile(act, q_d, s_d, 0)
    workspace = ext.wq_gemm_a16_tile_gate_up_silu(x, q_gu, s_gu, 0, n_down)
    prepared = workspace.view(torch.uint8)[: m * inter * 2].clone()
    got = ext.wq_gemm_a16_tile_prepared(workspace, m, q_d, s_d, 0)
    assert torch.equal(got, want)
    assert float(want.float().abs().mean()) > 0
    # the chunks: eight consecutive bf16 values in the order (0, 4, 1, 5, 2, 6, 3, 7)
    chunks = act.view(m, inter // 8, 8)[:, :, [0, 4, 1, 5, 2, 6, 3, 7]].contiguous()
    assert torch.equal(prepared, chunks.view(torch.uint8).flatten())
