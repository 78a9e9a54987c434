"""Finding, building and loading the gfx950 kernels.

Counterpart of llmquant/cuda/build.py in the reference, minus the JIT: the kernels are
compiled ahead of time, in-tree, by the Makefile one directory up (hipcc cross-compiles
gfx950 without a GPU), and this module only loads the result:

  libllmq_hip.so      the C ABI (include/llmq.h): kernels, plain pointers, a stream
  llmq_torch_ext.so   ATen/pybind layer exporting fake_quant_group, wq_gemv, ... on top of it

There is no fallback. If the extension is missing it is built; if that fails, or there is
no GPU, load_extension() raises.
"""

from __future__ import annotations

import ctypes
import functools
import importlib.util
import pathlib
import subprocess

HERE = pathlib.Path(__file__).resolve().parent
PACKAGE_ROOT = HERE.parent.parent  # the directory holding the Makefile and csrc/
CAPI_PATH = HERE / "libllmq_hip.so"
EXT_PATH = HERE / "llmq_torch_ext.so"
EXT_NAME = "llmq_torch_ext"


def build_extension(verbose: bool = False) -> None:
    """Compile both libraries for gfx950 with the in-tree Makefile. Always recompiles."""
    cmd = ["make", "-C", str(PACKAGE_ROOT), "-B", "-j8", "all"]
    result = subprocess.run(cmd, capture_output=not verbose, text=True)
    if result.returncode != 0:
        tail = "" if verbose else (result.stdout or "")[-2000:] + (result.stderr or "")[-4000:]
        raise RuntimeError(f"building the HIP kernels failed ({' '.join(cmd)}):\n{tail}")


def import_extension():
    """Load the prebuilt torch extension (no GPU needed just to load it)."""
    import torch  # noqa: F401  -- brings in libtorch and the HIP runtime the extension links to

    if not EXT_PATH.exists() or not CAPI_PATH.exists():
        raise RuntimeError(
            f"the HIP kernels are not built: {EXT_PATH} is missing. "
            f"Run `make -C {PACKAGE_ROOT}` (or __graft_entry__.build())."
        )
    spec = importlib.util.spec_from_file_location(EXT_NAME, str(EXT_PATH))
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return module


@functools.lru_cache(maxsize=1)
def load_extension(verbose: bool = False):
    """The extension module, loaded once per process. Raises without a GPU."""
    import torch

    if not torch.cuda.is_available():
        raise RuntimeError("CUDA is not available; the kernels need a GPU to run")
    if not EXT_PATH.exists() or not CAPI_PATH.exists():
        build_extension(verbose)
    return import_extension()


@functools.lru_cache(maxsize=1)
def load_capi() -> ctypes.CDLL:
    """The C ABI library through ctypes, with argument types declared. Loading needs no GPU."""
    import torch  # noqa: F401  -- so libamdhip64 resolves to the copy torch already loaded

    if not CAPI_PATH.exists():
        raise RuntimeError(f"{CAPI_PATH} is missing; run `make -C {PACKAGE_ROOT} capi`")
    lib = ctypes.CDLL(str(CAPI_PATH))
    c_int, c_i64, c_p, c_f = ctypes.c_int, ctypes.c_int64, ctypes.c_void_p, ctypes.c_float
    lib.llmq_abi_version.restype = c_int
    lib.llmq_last_error.restype = ctypes.c_char_p
    lib.llmq_fake_quant_group.argtypes = [c_p, c_p, c_p, c_i64, c_int, c_int, c_int, c_p]
    lib.llmq_quant_group_codes.argtypes = [c_p, c_p, c_p, c_i64, c_int, c_int, c_int, c_int, c_p]
    lib.llmq_wq_gemv.argtypes = [c_p, c_p, c_p, c_p] + [c_int] * 7 + [c_p]
    lib.llmq_kv_append.argtypes = [c_p, c_p, c_i64, c_i64, c_p, c_p, c_p, c_p, c_p, c_p, c_p] + [c_int] * 6 + [c_p]
    lib.llmq_kv_dequant.argtypes = [c_p, c_p, c_p] + [c_int] * 6 + [c_p]
    lib.llmq_kv_decode_workspace_floats.argtypes = [c_int] * 3
    lib.llmq_kv_decode_workspace_floats.restype = ctypes.c_size_t
    lib.llmq_kv_decode_attention.argtypes = [c_p] * 8 + [c_f] + [c_int] * 6 + [c_p]
    lib.llmq_kv_decode_attention_static.argtypes = [c_p] * 7 + [c_f] + [c_int] * 6 + [c_p]
    lib.llmq_kv_decode_attention_static.restype = c_int
    lib.llmq_wq_gemv_fused.argtypes = [c_p] * 4 + [c_int] * 6 + [c_p, c_f, c_int, c_p, c_p]
    lib.llmq_wq_gemv_fused.restype = c_int
    lib.llmq_wq_gemv_batched_fused.argtypes = [c_p, c_i64, c_p, c_p, c_p, c_p, c_p, c_p] + [c_int] * 8 + [c_p]
    lib.llmq_wq_gemv_batched_fused.restype = c_int
    lib.llmq_moe_combine.argtypes = [c_p] * 4 + [c_int] * 5 + [c_p]
    lib.llmq_moe_combine.restype = c_int
    lib.llmq_route_plan_blocks_per_expert.argtypes = [c_int, c_int]
    lib.llmq_route_plan_blocks_per_expert.restype = c_int
    lib.llmq_route_plan_supported.argtypes = [c_int, c_int]
    lib.llmq_route_plan_supported.restype = c_int
    lib.llmq_route_plan.argtypes = [c_p] + [c_int] * 3 + [c_p] * 5
    lib.llmq_route_plan.restype = c_int
    lib.llmq_wq_gemv_gate_up_silu.argtypes = [c_p] * 4 + [c_int] * 5 + [c_p, c_f, c_p]
    lib.llmq_wq_gemv_gate_up_silu.restype = c_int
    lib.llmq_kv_rope_append_attend.argtypes = [c_p] * 9 + [c_f] + [c_int] * 6 + [c_p]
    lib.llmq_kv_rope_append_attend.restype = c_int
    lib.llmq_kv_attend_partials_floats.argtypes = [c_int] * 3
    lib.llmq_kv_attend_partials_floats.restype = ctypes.c_size_t
    lib.llmq_kv_rope_append_attend_split.argtypes = [c_p] * 9 + [c_f] + [c_int] * 7 + [c_p]
    lib.llmq_kv_rope_append_attend_split.restype = c_int
    lib.llmq_kv_attend_merge.argtypes = [c_p, c_p] + [c_int] * 4 + [c_p]
    lib.llmq_kv_attend_merge.restype = c_int
    lib.llmq_wq_gemv_attn_merge.argtypes = [c_p, c_int, c_int, c_p, c_p, c_p] + [c_int] * 6 + [c_p, c_p]
    lib.llmq_wq_gemv_attn_merge.restype = c_int
    lib.llmq_dense_gemv_fused.argtypes = [c_p, c_p, c_p, c_int, c_int, c_int, c_int, c_p, c_f, c_p, c_int, c_int, c_int, c_p]
    lib.llmq_dense_gemv_fused.restype = c_int
    lib.llmq_argmax_row.argtypes = [c_p, c_int, c_p, c_int, c_p]
    lib.llmq_argmax_row.restype = c_int
    lib.llmq_argmax_advance.argtypes = [c_p, c_int, c_p, c_p, c_p, c_p, c_int, c_p]
    lib.llmq_argmax_advance.restype = c_int
    lib.llmq_prefill_attention.argtypes = [c_p, c_p, c_p, c_p, c_int, c_int, c_int, c_int, ctypes.c_float, c_int, c_p]
    lib.llmq_prefill_attention.restype = c_int
    lib.llmq_argmax_advance_embed.argtypes = [c_p, c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_int, c_p, c_int, c_p]
    lib.llmq_argmax_advance_embed.restype = c_int
    lib.llmq_argmax_workspace_bytes.argtypes = []
    lib.llmq_argmax_workspace_bytes.restype = ctypes.c_size_t
    lib.llmq_wq_gemm_a8.argtypes = [c_p] * 6 + [c_int] * 7 + [c_p]
    lib.llmq_wq_gemm_a8.restype = c_int
    lib.llmq_wq_gemm_a8_fast.argtypes = [c_p] * 7 + [ctypes.c_size_t] + [c_int] * 8 + [c_p]
    lib.llmq_wq_gemm_a8_fast.restype = c_int
    lib.llmq_wq_gemm_a8_fast_workspace_bytes.argtypes = [c_int] * 3
    lib.llmq_wq_gemm_a8_fast_workspace_bytes.restype = ctypes.c_size_t
    lib.llmq_act_codes_tiled_bytes.argtypes = [c_int] * 2
    lib.llmq_act_codes_tiled_bytes.restype = ctypes.c_size_t
    lib.llmq_quant_act_codes_tiled.argtypes = [c_p] * 3 + [c_int] * 4 + [c_p]
    lib.llmq_quant_act_codes_tiled.restype = c_int
    lib.llmq_wq_gemm_a8_tiled.argtypes = [c_p] * 6 + [c_int] * 7 + [c_p]
    lib.llmq_wq_gemm_a8_tiled.restype = c_int
    lib.llmq_wq_gemm_a8_takes_groups.argtypes = [c_int] * 3
    lib.llmq_wq_gemm_a8_takes_groups.restype = c_int
    lib.llmq_wq_gemm_a16.argtypes = [c_p] * 4 + [c_int] * 7 + [c_p]
    lib.llmq_wq_gemm_a16.restype = c_int
    lib.llmq_wq_gemm_a16_split.argtypes = [c_p] * 5 + [ctypes.c_size_t] + [c_int] * 7 + [c_p]
    lib.llmq_wq_gemm_a16_split.restype = c_int
    lib.llmq_wq_gemm_a16_tile.argtypes = [c_p] * 5 + [ctypes.c_size_t] + [c_int] * 7 + [c_p]
    lib.llmq_wq_gemm_a16_tile.restype = c_int
    lib.llmq_wq_gemm_a16_tile_workspace_bytes.argtypes = [c_int] * 3
    lib.llmq_wq_gemm_a16_tile_prepared_bytes.argtypes = [c_int] * 2
    lib.llmq_wq_gemm_a16_tile_prepared_bytes.restype = ctypes.c_size_t
    lib.llmq_wq_gemm_a16_tile_gate_up_silu.argtypes = ([c_p] * 4 + [ctypes.c_size_t, c_p, ctypes.c_size_t] + [c_int] * 7
                                                       + [c_p])
    lib.llmq_wq_gemm_a16_tile_gate_up_silu.restype = c_int
    lib.llmq_wq_gemm_a16_tile_gate_up_silu_prepared.argtypes = ([c_p] * 3 + [ctypes.c_size_t, c_p, ctypes.c_size_t]
                                                                + [c_int] * 7 + [c_p])
    lib.llmq_wq_gemm_a16_tile_gate_up_silu_prepared.restype = c_int
    lib.llmq_add_rmsnorm_prepared.argtypes = [c_p] * 5 + [ctypes.c_size_t, c_int, c_int, ctypes.c_float, c_int, c_p]
    lib.llmq_add_rmsnorm_prepared.restype = c_int
    lib.llmq_wq_gemm_a16_tile_prepared.argtypes = [c_p] * 4 + [ctypes.c_size_t] + [c_int] * 7 + [c_p]
    lib.llmq_wq_gemm_a16_tile_prepared.restype = c_int
    lib.llmq_wq_gemm_a16_tile_workspace_bytes.restype = ctypes.c_size_t
    lib.llmq_wq_gemm_a16_workspace_bytes.argtypes = [c_int] * 3
    lib.llmq_wq_gemm_a16_workspace_bytes.restype = ctypes.c_size_t
    lib.llmq_rmsnorm.argtypes = [c_p, c_p, c_p, c_int, c_int, ctypes.c_float, c_int, c_p]
    lib.llmq_rmsnorm.restype = c_int
    lib.llmq_add_rmsnorm.argtypes = [c_p] * 5 + [c_int, c_int, ctypes.c_float, c_int, c_p]
    lib.llmq_add_rmsnorm.restype = c_int
    lib.llmq_rope_qk.argtypes = [c_p] * 6 + [c_int] * 4 + [ctypes.c_int64] * 2 + [c_int, c_p]
    lib.llmq_rope_qk.restype = c_int
    lib.llmq_rope_kv_append.argtypes = ([c_p] * 3 + [ctypes.c_int64] * 3 + [c_p] * 10 + [c_int] * 7 + [c_p])
    lib.llmq_rope_kv_append.restype = c_int
    lib.llmq_silu_mul.argtypes = [c_p, c_p, c_p, ctypes.c_int64, c_int, c_p]
    lib.llmq_silu_mul.restype = c_int
    lib.llmq_silu_mul_rows.argtypes = [c_p, c_p, c_p, ctypes.c_int64, c_int, ctypes.c_int64, ctypes.c_int64, c_int, c_p]
    lib.llmq_silu_mul_rows.restype = c_int
    lib.llmq_wq_gemv_batched.argtypes = [c_p] * 7 + [c_int] * 9 + [c_p]
    lib.llmq_wq_gemv_batched.restype = c_int
    lib.llmq_wq_gemv_batched_max_rows.restype = c_int
    lib.llmq_dequant_weight.argtypes = [c_p, c_p, c_p] + [c_int] * 7 + [c_p]
    lib.llmq_dequant_weight.restype = c_int
    for name in ("llmq_fake_quant_group", "llmq_quant_group_codes", "llmq_wq_gemv", "llmq_kv_append",
                 "llmq_kv_dequant", "llmq_kv_decode_attention"):
        getattr(lib, name).restype = c_int
    return lib
