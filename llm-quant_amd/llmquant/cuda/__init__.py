"""Import-path parity with the reference: `from llmquant.cuda import load_extension,
fake_quantize_cuda` keeps working. Everything here is llmquant.hip."""

from llmquant.hip import fake_quantize_cuda, load_extension

__all__ = ["fake_quantize_cuda", "load_extension"]
