"""Running a quantized model: the integer KV cache, the kernel decode runtime, graphed decode."""

from llmquant.runtime.graph_decode import (WARMUP_CALLS, GraphedDecoder, KernelDecoder, can_graph, drop_kept,
                                           graphed_generate, kernel_runtime)
from llmquant.runtime.kv_cache import KernelQuantCache, make_kernel_cache_factory
from llmquant.runtime.llama_decode import LlamaKernelRuntime
from llmquant.runtime.llama_fused import LlamaDenseFusedRuntime, LlamaFusedRuntime

__all__ = ["WARMUP_CALLS", "GraphedDecoder", "KernelDecoder", "KernelQuantCache", "LlamaDenseFusedRuntime",
           "LlamaFusedRuntime", "LlamaKernelRuntime",
           "can_graph", "drop_kept", "graphed_generate", "kernel_runtime", "make_kernel_cache_factory"]
