"""Test configuration: import paths, the `gpu` marker, and shared helpers.

The package lives in llm-quant_amd/ (import name `llmquant`); the CPU oracle in oracle/.
Tests marked `gpu` need an MI355X and are deselected with -m "not gpu".
"""

import pathlib
import sys

import numpy as np
import pytest

ROOT = pathlib.Path(__file__).resolve().parent.parent
for extra in (ROOT / "llm-quant_amd", ROOT / "oracle", ROOT):
    if str(extra) not in sys.path:
        sys.path.insert(0, str(extra))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


DTYPE_TAGS = {"float32": "f32", "float16": "f16", "bfloat16": "bf16"}


def tag_of(torch_dtype) -> str:
    return DTYPE_TAGS[str(torch_dtype).removeprefix("torch.")]


def to_np(t) -> np.ndarray:
    """Any float tensor -> float32 numpy (exact: every storage type embeds in fp32)."""
    return t.detach().float().cpu().numpy()


def rel_l2(got, want) -> float:
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    return float(np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-30))
