#!/usr/bin/env python3
"""Benchmark of the `mode="kernel"` hot path on one MI355X.

A step is one pass of the weight-only GEMV (M = 1, bf16 activations) over every
Llama-3.2-1B linear shape -- q/o, k/v, gate/up, down and an untied lm_head -- each as int8
and as packed int4, symmetric group-128 weights quantized from bf16 N(0, 0.02). Inputs are
resident in HBM before the timed region; the weight buffers of successive steps rotate
through more than 512 MB so reads come from HBM, not from the 256 MB Infinity Cache.

Prints ONE JSON line. `value` is algorithmic GB/s over the whole step (real codes + fp32
scales + x + y; no padding bytes). `roofline` is the lm_head int8 launch alone, timed with
HIP events on the launch stream inside the timed region. `cpu_baseline` is the C oracle
(oracle/llmq_oracle.c, the reference's real-mode arithmetic) on the host cores, on the same
step. Extra keys report per-shape figures and the other kernels of the path.
"""

from __future__ import annotations

import argparse
import ctypes
import json
import os
import pathlib
import subprocess
import sys
import time

ROOT = pathlib.Path(__file__).resolve().parent
sys.path[:0] = [str(ROOT / "llm-quant_amd")]

GROUP = 128
HBM_PEAK_GBPS = 8000.0  # MI355X, published
SHAPES = [  # name, N, K  (BASELINE config 2)
    ("q/o", 2048, 2048),
    ("k/v", 512, 2048),
    ("gate/up", 8192, 2048),
    ("down", 2048, 8192),
    ("lm_head", 128256, 2048),
]


def algorithmic_bytes(n: int, k: int, bits: int, m: int = 1) -> int:
    """codes + fp32 scales + bf16 x + bf16 y."""
    return n * k * bits // 8 + n * (k // GROUP) * 4 + m * k * 2 + m * n * 2


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    return ap.parse_args()


def build_operands(torch, copies_bytes=600 << 20):
    """Quantize synthetic weights on the GPU with the package's own torch ops."""
    from llmquant.core.scheme import QuantizationArgs
    from llmquant.packing.packing import pack_int4
    from llmquant.quantizers.real import quantize_weight
    from llmquant.core.observers import group_view

    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(0)
    cases = []
    for name, n, k in SHAPES:
        w = (torch.randn(n, k, device=dev, generator=gen) * 0.02).to(torch.bfloat16)
        x = torch.randn(1, k, device=dev, generator=gen).to(torch.bfloat16)
        for bits in (8, 4):
            args = QuantizationArgs(num_bits=bits, strategy="group", group_size=GROUP)
            codes, scale = quantize_weight(w, args)
            canonical = group_view(codes, GROUP).contiguous()
            stored = pack_int4(canonical) if bits == 4 else canonical
            scales = scale.reshape(n, -1).contiguous().float()
            nbytes = algorithmic_bytes(n, k, bits)
            # enough rotating copies that one buffer is not touched again before > 512 MB
            # of other weights went by; rows are rolled so copies differ
            copies = 2 if nbytes > (64 << 20) else 3
            bufs = [(torch.roll(stored, i, 0).contiguous(), torch.roll(scales, i, 0).contiguous())
                    for i in range(copies)]
            cases.append(dict(name=name, n=n, k=k, bits=bits, x=x, bufs=bufs, bytes=nbytes,
                              out=torch.empty(1, n, device=dev, dtype=torch.bfloat16)))
        del w
    return cases


def main():
    opts = parse()
    if opts.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU form (see DESIGN.md, "
              "'How the path would shard'). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py needs an MI355X", file=sys.stderr)
        sys.exit(2)
    from llmquant.hip import load_capi, load_extension

    load_extension()
    lib = load_capi()
    torch.cuda.set_device(0)
    cases = build_operands(torch)
    stream = torch.cuda.current_stream()
    sptr = ctypes.c_void_p(stream.cuda_stream)
    BF16 = 2

    def launch(case, step):
        q, s = case["bufs"][step % len(case["bufs"])]
        rc = lib.llmq_wq_gemv(case["x"].data_ptr(), q.data_ptr(), s.data_ptr(), case["out"].data_ptr(),
                              1, case["n"], case["k"] // GROUP, GROUP, 0, case["bits"], BF16, sptr)
        if rc:
            raise RuntimeError(lib.llmq_last_error().decode())

    dominant = next(c for c in cases if c["name"] == "lm_head" and c["bits"] == 8)
    step_bytes = sum(c["bytes"] for c in cases)

    for step in range(opts.warmup):
        for case in cases:
            launch(case, step)
    torch.cuda.synchronize()

    # ---- timed region: exactly K steps; events bracket the dominant launch only
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
          for _ in range(opts.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for step in range(opts.steps):
        for case in cases:
            if case is dominant:
                ev[step][0].record(stream)
                launch(case, step)
                ev[step][1].record(stream)
            else:
                launch(case, step)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / opts.steps
    dom_ms = sorted(a.elapsed_time(b) for a, b in ev)
    dom_avg_ms = sum(dom_ms) / len(dom_ms)

    # ---- per-shape figures (outside the timed region): events around single launches
    shapes = []
    for case in cases:
        times = []
        for rep in range(30):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            # touch another ~0.5 GB first so this launch reads from HBM
            for other in cases:
                if other is not case and other["bytes"] > (100 << 20):
                    launch(other, rep)
            a.record(stream)
            launch(case, rep)
            b.record(stream)
            torch.cuda.synchronize()
            times.append(a.elapsed_time(b))
        times.sort()
        med = times[len(times) // 2]
        shapes.append({"shape": case["name"], "N": case["n"], "K": case["k"], "bits": case["bits"],
                       "bytes": case["bytes"], "us": round(med * 1e3, 2),
                       "GBps": round(case["bytes"] / (med * 1e-3) / 1e9, 1),
                       "frac_hbm": round(case["bytes"] / (med * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)})

    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    achieved = dominant["bytes"] / (dom_avg_ms * 1e-3) / 1e9
    result = {
        "metric": "W4/W8 GEMV HBM GB/s (% peak); 1B decode tok/s; W4A8 GEMM int8 TOPS",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": opts.steps,
        "warmup": opts.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "configs[1]: M=1 weight-only GEMV sweep over the five "
                               "Llama-3.2-1B linear shapes, int8 and packed int4, g128",
                   "bytes_per_step": step_bytes, "launches_per_step": len(cases)},
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBPS, 4),
        "roofline": {"bound": "hbm", "kernel": "wq_gemv lm_head 128256x2048 int8 M=1",
                     "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": None,
                     "avg_launch_us": round(dom_avg_ms * 1e3, 2),
                     "median_launch_us": round(dom_ms[len(dom_ms) // 2] * 1e3, 2),
                     "algorithmic_bytes": dominant["bytes"]},
        "shapes": shapes,
    }

    if not opts.no_cpu:
        result["cpu_baseline"] = cpu_baseline(torch, cases, opts.cpu_seconds)

    print(json.dumps(result))


def cpu_baseline(torch, cases, budget_s: float):
    """The C oracle (the reference's real-mode GEMV arithmetic) on the host cores, on the
    same operands, for about `budget_s` seconds."""
    lib_path = ROOT / "oracle" / "libllmq_oracle.so"
    if not lib_path.exists():
        subprocess.run(["make", "-C", str(ROOT / "oracle")], check=True, capture_output=True)
    olib = ctypes.CDLL(str(lib_path))
    olib.llmq_oracle_threads.restype = ctypes.c_int
    c_p, c_int = ctypes.c_void_p, ctypes.c_int
    olib.llmq_oracle_real_gemv_bf16.argtypes = [c_p, c_p, c_p, c_p] + [c_int] * 6
    olib.llmq_oracle_real_gemv_bf16.restype = None

    host = []
    for case in cases:
        q, s = case["bufs"][0]
        host.append((case, case["x"].cpu().view(torch.uint16).contiguous(), q.cpu().contiguous(),
                     s.cpu().contiguous(), torch.empty(1, case["n"], dtype=torch.float32)))
    step_bytes = sum(c["bytes"] for c in cases)

    def one_step():
        for case, x, q, s, out in host:
            olib.llmq_oracle_real_gemv_bf16(x.data_ptr(), q.data_ptr(), s.data_ptr(), out.data_ptr(),
                                            1, case["n"], case["k"] // GROUP, GROUP, 0,
                                            1 if case["bits"] == 4 else 0)

    one_step()
    t0 = time.perf_counter()
    steps = 0
    while time.perf_counter() - t0 < budget_s:
        one_step()
        steps += 1
    elapsed = time.perf_counter() - t0
    model = "unknown"
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    return {"value": round(step_bytes * steps / elapsed / 1e9, 2), "unit": "GB/s",
            "cores": int(olib.llmq_oracle_threads()), "kind": "port",
            "sample": f"{steps} full steps of the same sweep (same operands) in {elapsed:.1f} s, "
                      f"OpenMP over output rows",
            "cpu": model, "os_cpu_count": os.cpu_count()}


if __name__ == "__main__":
    main()
