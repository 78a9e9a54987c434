"""The three implementations of a quantized Linear and the lookup that picks one."""

from llmquant.quantizers.dispatch import AVAILABLE_MODES, quant_experts_for, quant_linear_for
from llmquant.quantizers.experts import KernelQuantExperts, RealQuantExperts, quantize_expert_stack, route_plan
from llmquant.quantizers.fake import FakeQuantCache, FakeQuantLinear, make_cache_factory
from llmquant.quantizers.kernel import FUSED_GEMM_MAX_ROWS, KERNEL_MAX_ROWS, KernelQuantLinear, pad_activation
from llmquant.quantizers.real import RealQuantLinear, exact_fp32_matmul, quantize_weight

__all__ = [
    "AVAILABLE_MODES", "FUSED_GEMM_MAX_ROWS", "KERNEL_MAX_ROWS", "FakeQuantCache", "FakeQuantLinear",
    "KernelQuantExperts", "KernelQuantLinear", "RealQuantExperts", "RealQuantLinear", "exact_fp32_matmul",
    "make_cache_factory", "pad_activation", "quant_experts_for", "quant_linear_for", "quantize_expert_stack",
    "quantize_weight", "route_plan",
]
