"""The integer prefill GEMM (int8 activations x int4/int8 weights) against the oracle's
real-mode forward: activation codes and scales bit-exact, outputs bit-exact (the kernel keeps
RealQuantLinear's rounding points and group order, llmquant/quantizers/real.py:94-99), at the
reference's own test size, ragged sizes, and the Llama-3.2-1B prefill shapes via sampled entries."""

import ctypes
import pathlib

import numpy as np
import pytest
import torch
import torch.nn as nn

import llmq_oracle as oracle
from conftest import rel_l2, tag_of, to_np

pytestmark = pytest.mark.gpu
GROUP = 128


@pytest.fixture(scope="module")
def ext():
    from llmquant.hip import load_extension

    return load_extension()


#: The exact GEMM has two bit-identical forms: tiled kernels that walk a tile's groups one after the other, and a
#: group-parallel kernel (eight groups of a 32 x 64 tile at once, additions in group order) for outputs of few
#: tiles. LLMQ_A8_FORM pins one whatever the shape; None is the library's own choice.
FORMS = pytest.mark.parametrize("form", ["tile", "groups", None], ids=["tiled", "group-parallel", "own choice"])


@pytest.fixture(autouse=True)
def no_form_left_pinned():
    import os

    yield
    os.environ.pop("LLMQ_A8_FORM", None)


def run_case(ext, m, n, k, bits, dtype, out_group=0, bias=False, seed=0, outliers=False, form=None):
    import os

    if form is None:
        os.environ.pop("LLMQ_A8_FORM", None)
    else:
        os.environ["LLMQ_A8_FORM"] = form
    torch.manual_seed(seed)
    w = (torch.randn(n, k) * 0.015).to(torch.bfloat16)
    x = torch.randn(m, k)
    if outliers:
        cols = torch.randperm(k)[: k // 100]
        x[:, cols] *= 20
    x = x.to(dtype)
    b = torch.randn(n) if bias else None
    canonical, scales = oracle.canonical_weight(to_np(w), bits, GROUP, None, out_group or None)
    q = torch.from_numpy(oracle.pack_int4(canonical) if bits == 4 else canonical).cuda()
    s = torch.from_numpy(scales).cuda()
    codes, sx = ext.quant_group_codes(x.cuda(), 8, GROUP, False)
    want_codes, want_sx = oracle.quant_group_codes(to_np(x), 8, GROUP)
    assert np.array_equal(codes.cpu().numpy(), want_codes) and np.array_equal(to_np(sx), want_sx)
    got = ext.wq_gemm_a8(codes, sx, q, s, b.cuda() if bias else None, out_group, dtype)
    return got, (x, canonical, scales, b)


@FORMS
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,n,k", [(32, 256, 512), (1, 128, 128), (37, 200, 384), (130, 129, 256), (4, 512, 2048),
                                   (65, 70, 1152), (33, 64, 2176)])
def test_bit_exact_against_real_mode(ext, bits, dtype, m, n, k, form):
    """(1152 and 2176: nine and seventeen groups, a last round of the group-parallel form with one group in it.)"""
    got, (x, canonical, scales, _) = run_case(ext, m, n, k, bits, dtype, form=form)
    want = oracle.real_linear(to_np(x), canonical, scales, tag_of(dtype), None, 8)
    assert got.shape == (m, n) and got.dtype == dtype
    assert np.array_equal(to_np(got).view(np.uint32), want.view(np.uint32))


@FORMS
@pytest.mark.parametrize("bits", [4, 8])
def test_bias_and_head_scales(ext, bits, form):
    got, (x, canonical, scales, b) = run_case(ext, 70, 192, 512, bits, torch.bfloat16, out_group=64, bias=True, seed=1,
                                              form=form)
    want = oracle.real_linear(to_np(x), canonical, scales, "bf16", 64, 8, to_np(b))
    assert np.array_equal(to_np(got), want)


def untile_codes(tiled, m, k, even_odd):
    """The [m, k] codes out of llmq_quant_act_codes_tiled's layout: blocks of 32 rows x one group, inside a block
    [k-step][row % 32 + 32 * k-half][16 bytes], with packed weights every eight bytes as even k then odd k."""
    padded = -(-m // 32) * 32
    t = tiled.reshape(padded // 32, k // GROUP, 4, 2, 32, 2, 8)      # m-tile, group, k-step, k-half, row, run, byte
    if even_odd:
        t = t[..., [0, 4, 1, 5, 2, 6, 3, 7]]
    t = t.transpose(0, 4, 1, 3, 2, 5, 6)                             # m-tile, row, group, k-half, k-step, run, byte
    return t.reshape(padded, k)[:m]


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,n,k", [(32, 256, 512), (1, 128, 128), (37, 200, 384), (130, 129, 256), (65, 70, 1152),
                                   (33, 64, 2176), (128, 512, 4096)])
def test_operand_order_codes_give_the_same_bits(ext, bits, dtype, m, n, k):
    """llmq_quant_act_codes_tiled + llmq_wq_gemm_a8_tiled: the scales and (taken out of the layout again) the codes of
    llmq_quant_group_codes, which are the oracle's; the product bit for bit the real-mode forward, with a bias and
    one weight scale row per 64 rows as well; rows of the last block of 32 that do not exist are never written."""
    torch.manual_seed(m + k)
    w = (torch.randn(n, k) * 0.015).to(torch.bfloat16)
    x = torch.randn(m, k).to(dtype)
    b = torch.randn(n)
    want_codes, want_sx = oracle.quant_group_codes(to_np(x), 8, GROUP)
    tiled, sx = ext.quant_act_codes_tiled(x.cuda(), bits)
    assert tiled.numel() == -(-m // 32) * 32 * k and np.array_equal(to_np(sx), want_sx)
    assert np.array_equal(untile_codes(tiled.cpu().numpy(), m, k, bits == 4), want_codes)
    for out_group, bias in ((0, None), (64, b)):
        canonical, scales = oracle.canonical_weight(to_np(w), bits, GROUP, None, out_group or None)
        q = torch.from_numpy(oracle.pack_int4(canonical) if bits == 4 else canonical).cuda()
        s = torch.from_numpy(scales).cuda()
        got = ext.wq_gemm_a8_tiled(tiled, sx, m, q, s, None if bias is None else bias.cuda(), out_group, dtype)
        want = oracle.real_linear(to_np(x), canonical, scales, tag_of(dtype), out_group or None, 8,
                                  None if bias is None else to_np(bias))
        assert got.shape == (m, n) and got.dtype == dtype
        assert np.array_equal(to_np(got), want)
        natural, _ = ext.quant_group_codes(x.cuda(), 8, GROUP, False)
        assert torch.equal(got, ext.wq_gemm_a8(natural, sx, q, s, None if bias is None else bias.cuda(), out_group, dtype))


def test_operand_order_at_the_long_row_shape_and_through_the_module(ext):
    """128 x 4096 x 14336 int4 (the shape the group-parallel kernel is for) on sampled entries against the oracle,
    and KernelQuantLinear with int8 activations taking that pair of calls for it (the natural-order calls are made
    to fail loudly), equal to RealQuantLinear's forward."""
    got, (x, canonical, scales, _) = run_case(ext, 128, 4096, 14336, 4, torch.bfloat16, seed=3, outliers=True)
    tiled, sx = ext.quant_act_codes_tiled(x.cuda(), 4)
    q = torch.from_numpy(oracle.pack_int4(canonical)).cuda()
    fast = ext.wq_gemm_a8_tiled(tiled, sx, 128, q, torch.from_numpy(scales).cuda(), None, 0, torch.bfloat16)
    assert torch.equal(fast, got) and ext.wq_gemm_a8_takes_groups(128, 4096, 112)
    assert not ext.wq_gemm_a8_takes_groups(2048, 4096, 112) and not ext.wq_gemm_a8_takes_groups(128, 14336, 32)
    import torch.nn as nn

    from llmquant.core.scheme import QuantizationArgs, QuantizationScheme
    from llmquant.quantizers import KernelQuantLinear, RealQuantLinear

    torch.manual_seed(5)
    linear = nn.Linear(4096, 1024, bias=True).to(torch.bfloat16).cuda()
    scheme = QuantizationScheme(weights=QuantizationArgs(num_bits=4, strategy="group", group_size=GROUP),
                                input_activations=QuantizationArgs(num_bits=8, strategy="group", group_size=GROUP))
    module, real = KernelQuantLinear.from_linear(linear, scheme), RealQuantLinear.from_linear(linear, scheme)
    xs = torch.randn(3, 40, 4096, device="cuda").to(torch.bfloat16)
    assert ext.wq_gemm_a8_takes_groups(120, 1024, 32)
    want = real(xs)

    class OnlyTiled:
        def __getattr__(self, name):
            if name in ("quant_group_codes", "wq_gemm_a8"):
                raise AssertionError(f"{name} called: the operand-order pair should have run")
            return getattr(ext, name)

    module._ext = OnlyTiled()
    assert torch.equal(module(xs), want)


def test_operand_order_argument_checks(ext):
    x = torch.randn(40, 256, device="cuda").to(torch.bfloat16)
    with pytest.raises(RuntimeError, match="bfloat16 or float16"):
        ext.quant_act_codes_tiled(x.float(), 4)
    with pytest.raises(RuntimeError, match="multiple of 128"):
        ext.quant_act_codes_tiled(x[:, :200].contiguous(), 4)
    tiled, sx = ext.quant_act_codes_tiled(x, 4)
    q = torch.randint(0, 256, (64, 2, 64), dtype=torch.uint8, device="cuda")
    s = torch.ones(64, 2, device="cuda")
    with pytest.raises(RuntimeError, match="not the codes of"):
        ext.wq_gemm_a8_tiled(tiled[:1024], sx, 40, q, s)
    with pytest.raises(RuntimeError, match="sx must be"):
        ext.wq_gemm_a8_tiled(tiled, sx[:, :1].contiguous(), 40, q, s)
    assert ext.wq_gemm_a8_tiled(tiled, sx, 40, q, s).shape == (40, 64)


def test_matches_the_float64_closed_form(ext):
    """Independent of the accumulation order: y = sum_g sx sw sum_k a q, in float64."""
    got, (x, canonical, scales, _) = run_case(ext, 64, 256, 1024, 4, torch.float32, seed=2)
    a, sx = oracle.quant_group_codes(to_np(x), 8, GROUP)
    xq = (a.reshape(64, -1, GROUP).astype(np.float64) * sx[..., None].astype(np.float64)).reshape(64, -1)
    exact = oracle.gemv_float64(xq, canonical, scales)
    assert rel_l2(to_np(got), exact) <= 1e-6


@pytest.mark.parametrize("form", ["tile", "groups"], ids=["tiled", "group-parallel"])
@pytest.mark.parametrize("n,k", [(14336, 4096), (4096, 14336)])
@pytest.mark.parametrize("m", [128, 512, 2048])
def test_llama_8b_mlp_shapes_on_sampled_entries(ext, n, k, m, form):
    """The 512-token prefill case at full size (1% outlier channels x20): 64 x 64 sampled outputs,
    bit-exact against the oracle restricted to those rows and columns, through both forms of the kernel."""
    got, (x, canonical, scales, _) = run_case(ext, m, n, k, 4, torch.bfloat16, seed=3, outliers=True, form=form)
    rng = np.random.default_rng(0)
    rows = np.sort(rng.choice(m, 64, replace=False))
    cols = np.sort(rng.choice(n, 64, replace=False))
    want = oracle.real_linear(to_np(x)[rows], canonical[cols], scales[cols], "bf16", None, 8)
    assert np.array_equal(to_np(got)[np.ix_(rows, cols)], want)


@pytest.mark.parametrize("bits", [4, 8])
def test_ragged_edges_of_the_large_tile(ext, bits):
    """Enough 128 x 128 tiles that the large-tile kernel runs, with M and N that end inside a
    tile: the last rows and columns (and a sample of the rest) against the oracle."""
    m, n, k = 2050, 3970, 256
    got, (x, canonical, scales, _) = run_case(ext, m, n, k, bits, torch.bfloat16, seed=4)
    rng = np.random.default_rng(1)
    rows = np.unique(np.concatenate([rng.choice(m, 48, replace=False), np.arange(m - 4, m)]))
    cols = np.unique(np.concatenate([rng.choice(n, 48, replace=False), np.arange(n - 4, n)]))
    want = oracle.real_linear(to_np(x)[rows], canonical[cols], scales[cols], "bf16", None, 8)
    assert np.array_equal(to_np(got)[np.ix_(rows, cols)], want)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("groups", [1, 3, 4, 5, 8, 9])
def test_large_tile_over_odd_and_even_group_counts(ext, bits, groups):
    """The large-tile kernel walks two groups a trip (one per LDS buffer) in a steady loop with no branches and
    finishes in a loop that has them: rows of 1 to 9 groups pass through every combination of the two (none, the
    tail alone, odd and even remainders) on an output that ends inside a tile, with both weight widths. The whole
    output must equal the group-parallel kernel's bit for bit, and sampled rows and columns the oracle's."""
    m, n, k = 2051, 2309, groups * GROUP   # 17 x 19 large tiles
    got, (x, canonical, scales, _) = run_case(ext, m, n, k, bits, torch.bfloat16, seed=groups, form="tile")
    other, _ = run_case(ext, m, n, k, bits, torch.bfloat16, seed=groups, form="groups")
    assert torch.equal(got, other)
    rng = np.random.default_rng(groups)
    rows = np.unique(np.concatenate([rng.choice(m, 40, replace=False), np.arange(m - 4, m)]))
    cols = np.unique(np.concatenate([rng.choice(n, 40, replace=False), np.arange(n - 6, n)]))
    want = oracle.real_linear(to_np(x)[rows], canonical[cols], scales[cols], "bf16", None, 8)
    assert np.array_equal(to_np(got)[np.ix_(rows, cols)], want)


@pytest.mark.parametrize("name", ["W4A8", "W8A8"])
@pytest.mark.parametrize("layout", [dict(), dict(head_dim=64), dict(out_group=64)])
@pytest.mark.parametrize("m", [1, 4, 33])
def test_module_equals_real_mode_on_device(name, layout, m):
    """KernelQuantLinear with an int8 activation scheme against RealQuantLinear run by torch on
    the same GPU (reference tests/test_kernel_linear.py's equality, for the A8 schemes)."""
    from dataclasses import replace

    from llmquant.core.scheme import QuantizationScheme, preset_name_to_scheme
    from llmquant.quantizers import KernelQuantLinear, RealQuantLinear

    base = preset_name_to_scheme(name)
    act = replace(base.input_activations, head_dim=layout["head_dim"]) if "head_dim" in layout else base.input_activations
    scheme = QuantizationScheme(weights=replace(base.weights, **layout), input_activations=act)
    torch.manual_seed(0)
    linear = nn.Linear(2048, 512, bias=True).cuda().to(torch.bfloat16)
    x = torch.randn(m, 2048, device="cuda", dtype=torch.bfloat16)
    module = KernelQuantLinear.from_linear(linear, scheme)
    got = module(x)
    want = RealQuantLinear.from_linear(linear, scheme)(x)
    assert got.shape == want.shape and torch.equal(got, want)
    # the module's switch to the fast form: same integer sums, one rounding fewer per group
    module.a8_exact = False
    fast = module(x)
    assert fast.shape == want.shape
    assert (fast == want).float().mean().item() > 0.98
    assert rel_l2(fast.detach().float().cpu().numpy(), want.detach().float().cpu().numpy()) <= 4e-3


def test_c_oracle_agrees_at_a_larger_size(ext):
    """The C restatement (also the timed CPU baseline) against the kernel, 256 x 1024 x 2048."""
    root = pathlib.Path(__file__).resolve().parent.parent
    lib = ctypes.CDLL(str(root / "oracle" / "libllmq_oracle.so"))
    got, (x, canonical, scales, _) = run_case(ext, 256, 1024, 2048, 4, torch.float32, seed=4)
    a, sx = oracle.quant_group_codes(to_np(x), 8, GROUP)
    packed = oracle.pack_int4(canonical)
    out = np.empty((256, 1024), dtype=np.float32)
    ptr = lambda arr: arr.ctypes.data_as(ctypes.c_void_p)
    lib.llmq_oracle_real_gemm_a8(ptr(a), ptr(np.ascontiguousarray(sx)), ptr(packed), ptr(scales), ptr(out),
                                 256, 1024, 16, 128, 0, 1)
    assert np.array_equal(to_np(got), out)


def test_argument_checks(ext):
    a = torch.zeros(4, 256, dtype=torch.int8, device="cuda")
    sx = torch.ones(4, 2, device="cuda")
    q = torch.zeros(8, 2, 128, dtype=torch.int8, device="cuda")
    s = torch.ones(8, 2, device="cuda")
    assert ext.wq_gemm_a8(a, sx, q, s).shape == (4, 8)
    with pytest.raises(RuntimeError, match="a must be int8"):
        ext.wq_gemm_a8(a.float(), sx, q, s)
    assert ext.wq_gemm_a8(a, sx[:, :1], q, s).shape == (4, 8)   # one scale per token
    with pytest.raises(RuntimeError, match="sx must be"):
        ext.wq_gemm_a8(a, torch.ones(4, 3, device="cuda"), q, s)
    with pytest.raises(RuntimeError, match="sx must be"):
        ext.wq_gemm_a8(a, torch.ones(4, 3, device="cuda"), q, s, None, 0, torch.float32, False)
    with pytest.raises(RuntimeError, match="group_size 128"):
        ext.wq_gemm_a8(a, torch.ones(4, 4, device="cuda"), torch.zeros(8, 4, 64, dtype=torch.int8, device="cuda"),
                       torch.ones(8, 4, device="cuda"))
    # the tiled kernels address a tile's rows with 32-bit offsets: rows beyond 2^24 codes are refused, not wrapped
    import os

    groups = (1 << 17) + 1
    os.environ["LLMQ_A8_FORM"] = "tile"
    with pytest.raises(RuntimeError, match="2\\^24 codes"):
        ext.wq_gemm_a8(torch.zeros(1, groups * 128, dtype=torch.int8, device="cuda"), torch.ones(1, groups, device="cuda"),
                       torch.zeros(1, groups, 128, dtype=torch.int8, device="cuda"), torch.ones(1, groups, device="cuda"))


@pytest.mark.parametrize("n,k", [(14336, 4096), (4096, 14336)])
@pytest.mark.parametrize("m", [128, 512, 2048])
def test_one_activation_scale_per_token(ext, n, k, m):
    """The prefill case with the activation quantized per token (one int8 scale per row, the literal
    "per-token symmetric int8"): the quantizer run with group = K, its scale broadcast to the [M, G] the
    kernel takes. The reference has no arithmetic of its own for this form (its activation scheme is per
    token x group-128, llmquant/core/scheme.py:41-44), so the anchor is the closed form
    y[m, n] = s_x[m] * sum_g s_w[n, g] * sum_k a[m, g, k] q[n, g, k] in float64 on sampled entries; codes and
    scales of the activation are bit-exact against the oracle's quantizer."""
    torch.manual_seed(7)
    w = (torch.randn(n, k) * 0.015).to(torch.bfloat16)
    x = torch.randn(m, k)
    x[:, torch.randperm(k)[: k // 100]] *= 20
    x = x.to(torch.bfloat16)
    canonical, scales = oracle.canonical_weight(to_np(w), 4, GROUP)
    q = torch.from_numpy(oracle.pack_int4(canonical)).cuda()
    s = torch.from_numpy(scales).cuda()
    codes, sx = ext.quant_group_codes(x.cuda(), 8, k, False)
    want_codes, want_sx = oracle.quant_group_codes(to_np(x), 8, k)
    assert sx.shape == (m, 1)
    assert np.array_equal(codes.cpu().numpy(), want_codes) and np.array_equal(to_np(sx), want_sx)
    sx_groups = sx.expand(m, k // GROUP).contiguous()
    rng = np.random.default_rng(2)
    rows = np.sort(rng.choice(m, 64, replace=False))
    cols = np.sort(rng.choice(n, 96, replace=False))
    a = want_codes[rows].astype(np.float64)
    wq = (canonical[cols].astype(np.float64) * scales[cols].astype(np.float64)[:, :, None]).reshape(len(cols), -1)
    exact = (a @ wq.T) * want_sx[rows].astype(np.float64)
    for dtype, tol in ((torch.float32, 1e-6), (torch.bfloat16, 1e-2)):
        got = ext.wq_gemm_a8(codes, sx_groups, q, s, None, 0, dtype)
        assert got.shape == (m, n) and got.dtype == dtype
        assert rel_l2(to_np(got)[np.ix_(rows, cols)], exact) <= tol
        # the fast form with the scale as [M, 1]: out of the sum over groups, applied once at the store
        fast = ext.wq_gemm_a8(codes, sx, q, s, None, 0, dtype, False)
        assert rel_l2(to_np(fast)[np.ix_(rows, cols)], exact) <= tol
        assert rel_l2(to_np(fast), to_np(got)) <= (1e-6 if dtype == torch.float32 else 4e-3)
        # (and the exact form takes [M, 1] too, broadcasting it itself)
        assert torch.equal(ext.wq_gemm_a8(codes, sx, q, s, None, 0, dtype), got)
    # against the unquantized product: what per-token int8 activations + int4 weights cost in accuracy
    dense = to_np(x)[rows].astype(np.float64) @ to_np(w)[cols].astype(np.float64).T
    print(f"per-token A8 x W4 vs bf16 product, M={m} N={n} K={k}: rel-L2 "
          f"{rel_l2(to_np(got)[np.ix_(rows, cols)], dense):.4f}")


# ---- the fast form: same integer sums, one rounding fewer per group, split reduction axis -------------------


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,n,k", [(128, 256, 128), (130, 300, 768), (1, 16, 128), (65, 257, 1152), (512, 512, 2048),
                                   (256, 1024, 8192)])
def test_fast_form_agrees_with_real_mode_to_fp32_rounding(ext, bits, dtype, m, n, k):
    """wq_gemm_a8(exact=False) against the oracle's real-mode forward and the float64 closed form: full and
    ragged tiles, one group, rows long enough that the reduction axis is split across workgroups."""
    torch.manual_seed(m + n)
    w = (torch.randn(n, k) * 0.015).to(torch.bfloat16)
    x = torch.randn(m, k)
    x[:, torch.randperm(k)[: max(k // 100, 1)]] *= 20
    x = x.to(torch.bfloat16)
    canonical, scales = oracle.canonical_weight(to_np(w), bits, GROUP)
    q = torch.from_numpy(oracle.pack_int4(canonical) if bits == 4 else canonical).cuda()
    s = torch.from_numpy(scales).cuda()
    codes, sx = ext.quant_group_codes(x.cuda(), 8, GROUP, False)
    got = ext.wq_gemm_a8(codes, sx, q, s, None, 0, dtype, False)
    assert got.shape == (m, n) and got.dtype == dtype
    a, sxo = oracle.quant_group_codes(to_np(x), 8, GROUP)
    xq = (a.reshape(m, -1, GROUP).astype(np.float64) * sxo[..., None].astype(np.float64)).reshape(m, -1)
    exact = oracle.gemv_float64(xq, canonical, scales)
    assert rel_l2(to_np(got), exact) <= (1e-6 if dtype == torch.float32 else 4e-3)
    real = oracle.real_linear(to_np(x), canonical, scales, tag_of(dtype), None, 8)
    if dtype == torch.float32:
        assert rel_l2(to_np(got), real) <= 1e-6
    else:
        assert (to_np(got) == real).mean() > 0.99
    # and against the bit-exact kernel on the same operands
    slow = ext.wq_gemm_a8(codes, sx, q, s, None, 0, dtype, True)
    assert rel_l2(to_np(got), to_np(slow)) <= (1e-6 if dtype == torch.float32 else 4e-3)


@pytest.mark.parametrize("bits", [4, 8])
def test_fast_form_bias_head_scales_and_split(ext, bits):
    torch.manual_seed(3)
    m, n, k = 70, 192, 8192   # one tile of long rows: the reduction axis is split, the bias is added by the second launch
    w = (torch.randn(n, k) * 0.015).to(torch.bfloat16)
    x = torch.randn(m, k).to(torch.bfloat16)
    b = torch.randn(n)
    canonical, scales = oracle.canonical_weight(to_np(w), bits, GROUP, None, 64)
    q = torch.from_numpy(oracle.pack_int4(canonical) if bits == 4 else canonical).cuda()
    codes, sx = ext.quant_group_codes(x.cuda(), 8, GROUP, False)
    got = ext.wq_gemm_a8(codes, sx, q, torch.from_numpy(scales).cuda(), b.cuda(), 64, torch.float32, False)
    want = oracle.real_linear(to_np(x), canonical, scales, "f32", 64, 8, to_np(b))
    assert rel_l2(to_np(got), want) <= 1e-6
    one = ext.wq_gemm_a8(codes[:, :512].contiguous(), sx[:, :4].contiguous(), q[:, :4].contiguous(),
                         torch.from_numpy(scales[:, :4].copy()).cuda(), b.cuda(), 64, torch.float32, False)
    want_one = oracle.real_linear(to_np(x)[:, :512], canonical[:, :4], scales[:, :4], "f32", 64, 8, to_np(b))
    assert rel_l2(to_np(one), want_one) <= 1e-6   # four groups: nothing is split, the bias added in the kernel


@pytest.mark.parametrize("n,k", [(14336, 4096), (4096, 14336)])
@pytest.mark.parametrize("m", [128, 2048])
def test_fast_form_at_llama_8b_mlp_shapes(ext, n, k, m):
    got, (x, canonical, scales, _) = run_case(ext, m, n, k, 4, torch.bfloat16, seed=3, outliers=True)
    codes, sx = ext.quant_group_codes(x.cuda(), 8, GROUP, False)
    q = torch.from_numpy(oracle.pack_int4(canonical)).cuda()
    fast = ext.wq_gemm_a8(codes, sx, q, torch.from_numpy(scales).cuda(), None, 0, torch.bfloat16, False)
    same = (fast == got).float().mean().item()
    assert same > 0.99 and rel_l2(to_np(fast), to_np(got)) <= 2e-3   # got: the bit-exact kernel


@pytest.mark.parametrize("bits", [4, 8])
def test_fast_form_one_scale_per_token_small_and_split(ext, bits):
    """One activation scale per token through the fast form on ragged tiles, with a bias, and on a shape whose
    reduction axis is split (the token's scale is applied to each partial tile)."""
    for m, n, k in ((70, 192, 8192), (130, 300, 768), (3, 40, 128)):
        torch.manual_seed(k)
        w = (torch.randn(n, k) * 0.015).to(torch.bfloat16)
        x = torch.randn(m, k).to(torch.bfloat16)
        b = torch.randn(n)
        canonical, scales = oracle.canonical_weight(to_np(w), bits, GROUP)
        q = torch.from_numpy(oracle.pack_int4(canonical) if bits == 4 else canonical).cuda()
        codes, sx = ext.quant_group_codes(x.cuda(), 8, k, False)
        want_codes, want_sx = oracle.quant_group_codes(to_np(x), 8, k)
        got = ext.wq_gemm_a8(codes, sx, q, torch.from_numpy(scales).cuda(), b.cuda(), 0, torch.float32, False)
        wq = (canonical.astype(np.float64) * scales.astype(np.float64)[:, :, None]).reshape(n, -1)
        exact = (want_codes.astype(np.float64) @ wq.T) * want_sx.astype(np.float64) + to_np(b).astype(np.float64)
        assert rel_l2(to_np(got), exact) <= 1e-6
