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
