"""Model loading (llmquant/core/model.py)."""

from llmquant.core.oneshot import load_pretrained

__all__ = ["load_pretrained"]
