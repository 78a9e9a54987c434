"""Latency measurement, deployed cost and the measured-versus-projected check, in the reference's row format."""

from llmquant.eval.cost import cost_columns, deployed_cost, kv_cache_bytes_per_token
from llmquant.eval.latency import latency_row, measure_latency
from llmquant.eval.verify import OUT_OF_KERNEL_AXES, PROJECTION_TOLERANCE, reconcile, verification_plan

__all__ = ["OUT_OF_KERNEL_AXES", "PROJECTION_TOLERANCE", "cost_columns", "deployed_cost", "kv_cache_bytes_per_token",
           "latency_row", "measure_latency", "reconcile", "verification_plan"]
