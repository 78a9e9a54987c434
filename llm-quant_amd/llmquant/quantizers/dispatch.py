"""`mode` -> module class (llmquant/quantizers/dispatch.py).

  fake    dequantize once, run the float Linear: what a dtype costs in accuracy
  real    keep the integers, multiply group by group in fp32: the reference arithmetic
  kernel  integers read by the HIP kernels: the deployed path
"""

AVAILABLE_MODES = frozenset({"fake", "real", "kernel"})


def quant_linear_for(mode: str):
    """Class that replaces each nn.Linear under `mode`. Imported lazily so llmquant.core
    never pulls a stage in at import time."""
    if mode not in AVAILABLE_MODES:
        raise ValueError(f"unsupported mode {mode!r}, expected one of {sorted(AVAILABLE_MODES)}")
    import llmquant.quantizers as stages

    return {"fake": stages.FakeQuantLinear, "real": stages.RealQuantLinear,
            "kernel": stages.KernelQuantLinear}[mode]


def quant_experts_for(mode: str):
    """Class that replaces a stacked Mixture-of-Experts block under `mode`, or None for "fake",
    which quantize-dequantizes the stacked parameters in place and keeps the block
    (llmquant/quantizers/dispatch.py:37-53)."""
    if mode not in AVAILABLE_MODES:
        raise ValueError(f"unsupported mode {mode!r}, expected one of {sorted(AVAILABLE_MODES)}")
    if mode == "fake":
        return None
    import llmquant.quantizers as stages

    return {"real": stages.RealQuantExperts, "kernel": stages.KernelQuantExperts}[mode]
