"""libllmq_hip.so loads on a machine without a GPU and exports every function include/llmq.h
declares; argument checks that need no device answer with an error code and a message."""

import ctypes
import pathlib
import re

import pytest

ROOT = pathlib.Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "llmq.h"


def declared_functions():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(llmq_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    from llmquant.hip.build import CAPI_PATH, load_capi

    if not CAPI_PATH.exists():
        from llmquant.hip.build import build_extension

        build_extension()
    return load_capi()


def test_header_declares_the_entry_points():
    names = declared_functions()
    for needed in ("llmq_abi_version", "llmq_last_error", "llmq_fake_quant_group", "llmq_quant_group_codes",
                   "llmq_wq_gemv"):
        assert needed in names


def test_every_declared_symbol_is_exported(lib):
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} is declared in include/llmq.h but not exported"
    assert lib.llmq_abi_version() == 1


def test_header_is_plain_c():
    import subprocess
    import tempfile

    with tempfile.TemporaryDirectory() as tmp:
        src = pathlib.Path(tmp) / "t.c"
        src.write_text('#include "llmq.h"\nint main(void) { return LLMQ_BF16 == 2 ? 0 : 1; }\n')
        subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-fsyntax-only", f"-I{HEADER.parent}", str(src)], check=True)


def test_argument_checks_need_no_device(lib):
    assert lib.llmq_fake_quant_group(None, None, None, 4, 128, 9, 2, None) == 1
    assert b"num_bits" in lib.llmq_last_error()
    assert lib.llmq_fake_quant_group(None, None, None, 4, 0, 8, 2, None) == 1
    assert b"group_size" in lib.llmq_last_error()
    assert lib.llmq_fake_quant_group(None, None, None, 0, 128, 8, 2, None) == 0  # empty input: nothing to do
    assert lib.llmq_wq_gemv(None, None, None, None, 1, 8, 1, 128, 0, 5, 2, None) == 1
    assert b"weight format" in lib.llmq_last_error()
    assert lib.llmq_wq_gemv(None, None, None, None, 1, 8, 1, 126, 0, 8, 2, None) == 1
    assert lib.llmq_wq_gemv(None, None, None, None, 0, 8, 1, 128, 0, 8, 2, None) == 0  # M == 0
    assert lib.llmq_quant_group_codes(None, None, None, 4, 128, 8, 1, 2, None) == 1
    assert b"null tensor pointer" in lib.llmq_last_error()


def test_fused_gemm_argument_checks_need_no_device(lib):
    # (x, qweight, wscale, out, M, N, G, gs, out_group, wformat, dtype, stream)
    assert lib.llmq_wq_gemm_a16(None, None, None, None, 8, 256, 4, 64, 0, 4, 2, None) == 1
    assert b"group_size 128" in lib.llmq_last_error()
    assert lib.llmq_wq_gemm_a16(None, None, None, None, 8, 256, 4, 128, 0, 4, 0, None) == 1
    assert b"float16 or bfloat16" in lib.llmq_last_error()
    assert lib.llmq_wq_gemm_a16(None, None, None, None, 8, 256, 4, 128, 0, 5, 2, None) == 1
    assert b"weight format" in lib.llmq_last_error()
    assert lib.llmq_wq_gemm_a16(None, None, None, None, 8, 256, 4, 128, -1, 4, 2, None) == 1
    assert b"out_group" in lib.llmq_last_error()
    assert lib.llmq_wq_gemm_a16(None, None, None, None, 8, 256, 0, 128, 0, 4, 2, None) == 1
    assert b"no groups" in lib.llmq_last_error()
    assert lib.llmq_wq_gemm_a16(None, None, None, None, 8, 256, 4, 128, 0, 4, 2, None) == 1
    assert b"null tensor pointer" in lib.llmq_last_error()
    assert lib.llmq_wq_gemm_a16(None, None, None, None, 0, 256, 4, 128, 0, 4, 2, None) == 0  # no rows: nothing to do

    # the reduction-axis form: (x, qweight, wscale, out, workspace, workspace_bytes, M, N, G, gs, ...)
    assert lib.llmq_wq_gemm_a16_split(None, None, None, None, None, 0, 8, 256, 4, 64, 0, 4, 2, None) == 1
    assert b"group_size 128" in lib.llmq_last_error()
    assert lib.llmq_wq_gemm_a16_split(None, None, None, None, None, 0, 8, 256, 4, 128, 0, 4, 0, None) == 1
    assert b"float16 or bfloat16" in lib.llmq_last_error()
    assert lib.llmq_wq_gemm_a16_split(None, None, None, None, None, 0, 8, 0, 4, 128, 0, 4, 2, None) == 0


def test_fused_gemm_workspace_is_one_fp32_tile_per_slice_of_four_groups(lib):
    size = lib.llmq_wq_gemm_a16_workspace_bytes
    assert size(16, 4096, 4) == 0                       # one slice writes the output itself
    assert size(16, 4096, 32) == 8 * 16 * 4096 * 4      # 32 groups = 8 slices of 4
    assert size(16, 4096, 33) == 9 * 16 * 4096 * 4      # a ragged last slice still has its tile
    assert size(200, 4096, 32) == 8 * 64 * 4096 * 4     # more than 64 rows go through in slabs of 64
    assert size(0, 4096, 32) == 0 and size(16, 0, 32) == 0 and size(16, 4096, 0) == 0


def test_prompt_pass_argument_checks_need_no_device(lib):
    # (x, weight, out, rows, hidden, eps, dtype, stream)
    assert lib.llmq_rmsnorm(None, None, None, 4, 0, 1e-5, 2, None) == 1
    assert b"bad dimension" in lib.llmq_last_error()
    assert lib.llmq_rmsnorm(None, None, None, 4, 2048, 1e-5, 7, None) == 1
    assert b"float32, float16 or bfloat16" in lib.llmq_last_error()
    assert lib.llmq_rmsnorm(None, None, None, 4, 2044, 1e-5, 2, None) == 1
    assert b"hidden must be a multiple of 8" in lib.llmq_last_error()
    assert lib.llmq_rmsnorm(None, None, None, 4, 2044, 1e-5, 0, None) == 1   # fp32 packets hold four: 2044 passes that check
    assert b"null tensor pointer" in lib.llmq_last_error()
    # (q, k, cos, sin, q_out, k_out, tokens, q_heads, kv_heads, head_dim, q_row_stride, k_row_stride, dtype, stream)
    assert lib.llmq_rope_qk(None, None, None, None, None, None, 4, 32, 8, 60, 1920, 480, 2, None) == 1
    assert b"head_dim must be a multiple of 16" in lib.llmq_last_error()
    assert lib.llmq_rope_qk(None, None, None, None, None, None, 4, 32, 8, 64, 2050, 512, 2, None) == 1
    assert b"row strides" in lib.llmq_last_error()
    assert lib.llmq_rope_qk(None, None, None, None, None, None, 4, 32, 8, 64, 2048, 512, 2, None) == 1
    assert b"null tensor pointer" in lib.llmq_last_error()
    # (gate, up, out, count, dtype, stream) and (gate, up, out, rows, width, gate_row_stride, up_row_stride, dtype, stream)
    assert lib.llmq_silu_mul(None, None, None, 12, 2, None) == 1
    assert b"multiple of 8" in lib.llmq_last_error()
    assert lib.llmq_silu_mul(None, None, None, -8, 2, None) == 1
    assert b"negative" in lib.llmq_last_error()
    assert lib.llmq_silu_mul_rows(None, None, None, 4, 8192, 16388, 16384, 2, None) == 1
    assert b"row strides" in lib.llmq_last_error()
    assert lib.llmq_silu_mul_rows(None, None, None, 4, 8192, 16384, 16384, 2, None) == 1
    assert b"null tensor pointer" in lib.llmq_last_error()


def test_rope_and_append_argument_checks_need_no_device(lib):
    # (q, k, v, q_row_stride, k_row_stride, v_row_stride, cos, sin, q_out, k_codes, v_codes, k_scale, v_scale,
    #  dq_k, dq_v, pos, tokens, q_heads, kv_heads, head_dim, t_max, bits, dtype, stream)
    nulls = [None] * 3 + [3072] * 3 + [None] * 10
    assert lib.llmq_rope_kv_append(*nulls, 4, 32, 8, 64, 16, 6, 2, None) == 1
    assert b"bits must be 8 or 4" in lib.llmq_last_error()
    assert lib.llmq_rope_kv_append(*nulls, 4, 32, 8, 96, 16, 8, 2, None) == 1
    assert b"head_dim must be 64 or 128" in lib.llmq_last_error()
    assert lib.llmq_rope_kv_append(*nulls, 4, 32, 8, 64, 16, 8, 9, None) == 1
    assert b"dtype" in lib.llmq_last_error()
    assert lib.llmq_rope_kv_append(*nulls, 4, 32, 8, 64, 16, 8, 2, None) == 1
    assert b"null tensor pointer" in lib.llmq_last_error()
    assert lib.llmq_rope_kv_append(*nulls, 0, 32, 8, 64, 16, 8, 2, None) == 0   # no tokens: nothing to do
