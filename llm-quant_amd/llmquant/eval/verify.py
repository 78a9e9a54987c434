"""Measure what a sweep only projected (llmquant/eval/verify.py:30-100): the selected recipe is
re-measured on the deployed path beside a bf16 baseline, and every axis whose work the weight
kernels do not do gets an ablation run with that axis back at bf16; the gap is that axis's cost.
"""

from __future__ import annotations

from dataclasses import replace

from llmquant.core.config import QuantConfig, normalize_dtype

BF16 = "bf16"
#: axes the analytic decode-traffic estimate cannot price, because their work is outside the GEMV
OUT_OF_KERNEL_AXES = ("kv_cache", "activation")
#: below this fraction of the projection, the projection is reported as not having held up
PROJECTION_TOLERANCE = 0.85


def verification_plan(quant: QuantConfig, winner_row: dict | None = None):
    """[(label, QuantConfig or None)]: the bf16 baseline (None), the selected recipe, and one
    ablation per out-of-kernel axis that is not bf16 already. Every run is meant to be driven
    the same way (graph replay on both sides), so the comparison prices the recipe alone."""
    if winner_row:
        quant = replace(quant, **{axis: winner_row[axis] for axis in
                                  ("attn_weight", "mlp_weight", "head_weight", "activation", "kv_cache")})
    plan = [("bf16 baseline", None), ("selected", quant)]
    for axis in OUT_OF_KERNEL_AXES:
        if normalize_dtype(getattr(quant, axis)) != BF16:
            plan.append((f"selected, {axis}=bf16", replace(quant, **{axis: BF16})))
    return plan


def reconcile(rows) -> dict:
    """Projection against measurement. `rows` carry `verify_label` and `decode_tps`; the selected
    row may carry `decode_speedup_projected`."""
    by_label = {r["verify_label"]: r for r in rows}
    baseline, selected = by_label.get("bf16 baseline"), by_label.get("selected")
    if not baseline or not selected or not baseline.get("decode_tps") or not selected.get("decode_tps"):
        return {}
    measured = selected["decode_tps"] / baseline["decode_tps"]
    projected = selected.get("decode_speedup_projected")
    result = {
        "measured_decode_speedup": measured,
        "projected_decode_speedup": projected,
        "baseline_tps": baseline["decode_tps"],
        "selected_tps": selected["decode_tps"],
        "held_up": None if not projected else measured >= projected * PROJECTION_TOLERANCE,
        "attribution": [],
    }
    for key, name in (("ttft_ms", "ttft_ratio"), ("peak_vram_gb", "vram_ratio")):
        if baseline.get(key) and selected.get(key):
            result[name] = selected[key] / baseline[key]
    # what putting one axis back at bf16 recovers
    for axis in OUT_OF_KERNEL_AXES:
        ablation = by_label.get(f"selected, {axis}=bf16")
        if not ablation or not ablation.get("decode_tps"):
            continue
        result["attribution"].append({
            "axis": axis,
            "dtype": normalize_dtype(selected.get(axis)),
            "tps_without_it": ablation["decode_tps"],
            "recovered": ablation["decode_tps"] / selected["decode_tps"],
            "costs_decode_pct": (1 - selected["decode_tps"] / ablation["decode_tps"]) * 100,
        })
    result["attribution"].sort(key=lambda a: -a["recovered"])
    return result
