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
SHAPES = [  # name, N, K  (the linear layers of Llama-3.2-1B and its lm_head)
    ("q/o", 2048, 2048),
    ("k/v", 512, 2048),
    ("gate/up", 8192, 2048),
    ("down", 2048, 8192),
    ("lm_head", 128256, 2048),
]


# HBM bytes one lm_head int8 launch moves, from hardware counters (FETCH_SIZE and WRITE_SIZE, each
# scaled by its reading for a 256 MiB copy): profiles/wq_gemv_lm_head_hbm_traffic.txt. 1.001 x the
# algorithmic bytes.
LM_HEAD_INT8_TRAFFIC_BYTES = 271_451_500


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
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the legs that report the path's other kernels and end-to-end decode")
    ap.add_argument("--only", choices=("other", "decode", "prefill", "decode8b"), default=None,
                    help="profiling aid: run just that leg and print its JSON (not the bench line)")
    ap.add_argument("--prompt-tokens", type=int, default=512, help="prompt length of the --only prefill leg")
    ap.add_argument("--copy-probe", action="store_true",
                    help="first run a plain 256 MiB device copy three times: the known-size kernel that "
                         "hardware-counter readings of the sweep are scaled by")
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
        print("bench.py measures one GPU: this path has no multi-GPU form (it would shard by output rows, "
              "kv heads and experts, with no exchange inside a kernel). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py needs an MI355X", file=sys.stderr)
        sys.exit(2)
    from llmquant.hip import load_capi, load_extension

    load_extension()
    lib = load_capi()
    torch.cuda.set_device(0)
    if opts.only:
        leg = {"other": other_kernels, "decode": decode_leg, "prefill": lambda t: prefill_leg(t, opts.prompt_tokens),
               "decode8b": lambda t: decode_leg(t, arch="llama3-8b")}[opts.only](torch)
        print(json.dumps({opts.only: leg}))
        return
    if opts.copy_probe:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda:0").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
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

    # ---- what a kernel that only reads gets out of this GPU's memory: 1 GiB per launch, rotating over 2 GiB
    probe = [torch.empty(1 << 30, dtype=torch.uint8, device="cuda:0").random_(0, 255) for _ in range(2)]
    sink = torch.zeros(1, dtype=torch.int32, device="cuda:0")
    probe_ms = []
    # (the probe kernel is a measurement aid in a small library of its own, beside the product library)
    probe_lib = ctypes.CDLL(str(ROOT / "llm-quant_amd" / "llmquant" / "hip" / "libllmq_bench_probe.so"))
    probe_lib.bench_stream_read_probe.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p]
    probe_lib.bench_stream_read_probe.restype = ctypes.c_int
    for rep in range(12):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record(stream)
        rc = probe_lib.bench_stream_read_probe(probe[rep % 2].data_ptr(), probe[rep % 2].numel(), sink.data_ptr(), sptr)
        b.record(stream)
        torch.cuda.synchronize()
        if rc:
            raise RuntimeError(f"bench_stream_read_probe: hipError {rc}")
        if rep >= 2:
            probe_ms.append(a.elapsed_time(b))
    read_ceiling = (1 << 30) / (sum(probe_ms) / len(probe_ms) * 1e-3) / 1e9
    del probe

    # ---- the roofline kernel again, as a decode loop runs it: back-to-back launches replayed from a graph
    def dominant_burst():
        here = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)  # the capturing stream
        for rep in range(12):
            q, s = dominant["bufs"][rep % len(dominant["bufs"])]
            rc = lib.llmq_wq_gemv(dominant["x"].data_ptr(), q.data_ptr(), s.data_ptr(), dominant["out"].data_ptr(),
                                  1, dominant["n"], dominant["k"] // GROUP, GROUP, 0, dominant["bits"], BF16, here)
            if rc:
                raise RuntimeError(lib.llmq_last_error().decode())

    dom_graph_us = _graph_time_us(torch, dominant_burst, reps=5) / 12

    # ---- configs[0]: the single down_proj int4 GEMV (2048 x 8192, M = 1) on its own line: the launch under graph
    # replay, weights rotated over > 600 MB (72 copies of 8.9 MB) so that every launch reads HBM
    down4 = next(c for c in cases if c["name"] == "down" and c["bits"] == 4)
    rot = [(torch.roll(down4["bufs"][0][0], i, 0).contiguous(), torch.roll(down4["bufs"][0][1], i, 0).contiguous())
           for i in range(72)]

    def config1_burst():
        here = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        for q, s in rot:
            rc = lib.llmq_wq_gemv(down4["x"].data_ptr(), q.data_ptr(), s.data_ptr(), down4["out"].data_ptr(),
                                  1, down4["n"], down4["k"] // GROUP, GROUP, 0, 4, BF16, here)
            if rc:
                raise RuntimeError(lib.llmq_last_error().decode())

    config1_us = _graph_time_us(torch, config1_burst, reps=5) / len(rot)
    del rot

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
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": LM_HEAD_INT8_TRAFFIC_BYTES,
                     "avg_launch_us": round(dom_avg_ms * 1e3, 2),
                     "median_launch_us": round(dom_ms[len(dom_ms) // 2] * 1e3, 2),
                     "algorithmic_bytes": dominant["bytes"],
                     "graph_replay_launch_us": round(dom_graph_us, 2),
                     "graph_replay_GBps": round(dominant["bytes"] / dom_graph_us / 1e3, 1),
                     "box_streaming_read_GBps": round(read_ceiling, 1),
                     "frac_of_box_streaming_read": round(achieved / read_ceiling, 4)},
        "shapes": shapes,
        "config1_down_proj_int4_gemv": {
            "workload": "configs[0]: N=2048, K=8192, M=1, int4 g128, bf16 activation, fp32 accumulation",
            "bytes": down4["bytes"], "graph_replay_launch_us": round(config1_us, 2),
            "GBps": round(down4["bytes"] / config1_us / 1e3, 1),
            "frac_hbm": round(down4["bytes"] / config1_us / 1e3 / HBM_PEAK_GBPS, 4),
            "note": "8.9 MB at 8 TB/s is 1.1 us, under the 2.0 us an empty kernel takes under graph replay: this "
                    "launch is bound by its fixed cost (launch, activation staging, first-byte latency), not by HBM"},
    }

    del cases
    torch.cuda.empty_cache()
    if not opts.no_extras:
        result["other_kernels"] = other_kernels(torch)
        result["decode"] = decode_leg(torch)

    if not opts.no_cpu:
        cases = build_operands(torch)
        result["cpu_baseline"] = cpu_baseline(torch, cases, opts.cpu_seconds)

    print(json.dumps(result))


def _event_time_us(torch, fn, reps=20, warm=3):
    for _ in range(warm):
        fn()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / reps * 1e3


_CAPI = {}


def _graph_time_us(torch, fn, reps=20):
    """Average replay time of `fn` captured as one HIP graph (launch cost of the Python loop removed)."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        fn()
    return _event_time_us(torch, graph.replay, reps=reps)


def other_kernels(torch):
    """The path's other kernels, each on the shape the reference quotes it on: fake-quant op, KV-cache decode
    step (config 4), W4A8 / W8A8 integer GEMM (config 3). Back-to-back launches, HIP events."""
    from llmquant.hip import load_extension

    from llmquant.hip import load_capi

    ext = load_extension()
    _CAPI["lib"] = load_capi()
    dev = "cuda:0"
    out = {}
    # fake quant, 2048 x 8192 bf16, g128: one read + one write (+ scales)
    xs = [torch.randn(2048, 8192, device=dev).to(torch.bfloat16) for _ in range(12)]  # 400 MB rotation
    i = [0]

    def fq():
        ext.fake_quant_group(xs[i[0] % len(xs)], 4, GROUP, True)
        i[0] += 1

    us = _event_time_us(torch, fq, reps=48)
    nbytes = 2 * 2048 * 8192 * 2 + 2048 * 64 * 4
    # what a plain device copy of the same tensors takes (one read + one write of the same bytes, no scales)
    ys = [torch.empty_like(x) for x in xs]

    def copy():
        ys[i[0] % len(xs)].copy_(xs[i[0] % len(xs)])
        i[0] += 1

    us_copy = _event_time_us(torch, copy, reps=48)
    out["fake_quant_2048x8192_bf16_int4"] = {"us": round(us, 2), "GBps": round(nbytes / us / 1e3, 1),
                                             "frac_hbm": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4),
                                             "device_copy_of_the_same_tensor_us": round(us_copy, 2)}
    del xs, ys
    # KV cache decode step, Llama-3.2-1B geometry, 2048 tokens of context + the one being decoded:
    # RoPE + quantize-and-append + attention in one launch per layer, 16 layers replayed as a graph
    # (16 layers of cache are 36 MB and would sit in the 256 MB Infinity Cache: the launches walk as many
    # layers' worth of cache as it takes to touch 300 MB, so every launch reads its cache from HBM)
    for bits in (8, 4):
        kvh, qh, d, t_max = 8, 32, 64, 2304
        layers = 128 if bits == 8 else 256
        ctx = 2048
        width = d if bits == 8 else d // 2
        dt = torch.int8 if bits == 8 else torch.uint8
        kc = torch.randint(0, 100, (layers, kvh, t_max, width), device=dev).to(dt)
        vc = torch.randint(0, 100, (layers, kvh, t_max, width), device=dev).to(dt)
        ks = torch.rand(layers, kvh, t_max, device=dev) * 0.05
        vs = torch.rand(layers, kvh, t_max, device=dev) * 0.05
        qkv = torch.randn(1, (qh + 2 * kvh) * d, device=dev).to(torch.bfloat16)
        table = torch.randn(t_max, d, device=dev).to(torch.bfloat16)
        pos = torch.tensor([ctx], dtype=torch.int32, device=dev)

        splits = 8
        partials = torch.zeros(ext.kv_attend_partials_floats(qh, d, splits), device=dev)

        def one_workgroup_per_head():
            for layer in range(layers):
                ext.kv_rope_append_attend(qkv, table, table, kc[layer], vc[layer], ks[layer], vs[layer], pos,
                                          d ** -0.5, qh)

        def split_only():  # in a decode step the records are merged by o_proj's GEMV, at no launch
            for layer in range(layers):
                ext.kv_rope_append_attend_split(qkv, table, table, kc[layer], vc[layer], ks[layer], vs[layer],
                                                partials, pos, d ** -0.5, qh, splits)

        def split_and_merge():
            for layer in range(layers):
                ext.kv_rope_append_attend_split(qkv, table, table, kc[layer], vc[layer], ks[layer], vs[layer],
                                                partials, pos, d ** -0.5, qh, splits)
                ext.kv_attend_merge(partials, qh, d, splits, torch.bfloat16)

        nbytes = 2 * kvh * (ctx + 1) * width + 2 * kvh * (ctx + 1) * 4
        entry = {"bytes": nbytes, "splits": splits, "layers_of_cache_walked": layers,
                 "cache_bytes_touched_per_replay": nbytes * layers}
        partials7 = torch.zeros(ext.kv_attend_partials_floats(qh, d, 7), device=dev)

        def vector_alu_7_splits():  # (below 8 splits the entry point keeps one head a workgroup on the vector ALU)
            for layer in range(layers):
                ext.kv_rope_append_attend_split(qkv, table, table, kc[layer], vc[layer], ks[layer], vs[layer],
                                                partials7, pos, d ** -0.5, qh, 7)

        # split_us: what the runtime's step runs on a cache of this size, 8 splits, four heads of a kv head a workgroup
        # with the cache's codes as matrix-core operands
        for name, fn in (("one_workgroup_per_head_us", one_workgroup_per_head), ("split_us", split_only),
                         ("split_plus_merge_kernel_us", split_and_merge),
                         ("vector_alu_7_splits_us", vector_alu_7_splits)):
            entry[name] = round(_graph_time_us(torch, fn, reps=5) / layers, 2)
        entry["GBps"] = round(nbytes / entry["split_us"] / 1e3, 1)
        out[f"kv_int{bits}_rope_append_attention_ctx2048_per_layer"] = entry
    # the same step on a long cache (32 000 tokens, int8; 10 layers = 350 MB, so that every launch reads HBM): one
    # query head per workgroup on the vector ALU (7 splits; from 8 on the entry point takes the other form) against
    # the form long caches take, four heads of a kv head per workgroup with the int8 codes as matrix-core operands
    layers, kvh, qh, d, t_max, ctx = 10, 8, 32, 64, 32768, 32000
    kc = torch.randint(0, 100, (layers, kvh, t_max, d), device=dev).to(torch.int8)
    vc = torch.randint(0, 100, (layers, kvh, t_max, d), device=dev).to(torch.int8)
    ks = torch.rand(layers, kvh, t_max, device=dev) * 0.05
    vs = torch.rand(layers, kvh, t_max, device=dev) * 0.05
    qkv = torch.randn(1, (qh + 2 * kvh) * d, device=dev).to(torch.bfloat16)
    table = torch.randn(t_max, d, device=dev).to(torch.bfloat16)
    pos = torch.tensor([ctx], dtype=torch.int32, device=dev)
    nbytes = 2 * kvh * (ctx + 1) * d + 2 * kvh * (ctx + 1) * 4
    entry = {"bytes": nbytes}
    for name, splits in (("one_head_per_workgroup_vector_alu_7_splits_us", 7), ("four_heads_matrix_core_32_splits_us", 32)):
        partials = torch.zeros(ext.kv_attend_partials_floats(qh, d, splits), device=dev)

        def long_step():
            for layer in range(layers):
                ext.kv_rope_append_attend_split(qkv, table, table, kc[layer], vc[layer], ks[layer], vs[layer],
                                                partials, pos, d ** -0.5, qh, splits)

        entry[name] = round(_graph_time_us(torch, long_step, reps=20) / layers, 2)
    entry["GBps"] = round(nbytes / entry["four_heads_matrix_core_32_splits_us"] / 1e3, 1)
    entry["frac_hbm"] = round(entry["GBps"] / HBM_PEAK_GBPS, 4)
    out["kv_int8_rope_append_attention_ctx32000_per_layer"] = entry
    del kc, vc, ks, vs
    # 131 000 tokens (3 layers = 430 MB): the cache's bytes are most of the launch
    layers, t_long, ctx_long = 3, 131072, 131000
    kc = torch.randint(0, 100, (layers, kvh, t_long, d), device=dev).to(torch.int8)
    vc = torch.randint(0, 100, (layers, kvh, t_long, d), device=dev).to(torch.int8)
    ks = torch.rand(layers, kvh, t_long, device=dev) * 0.05
    vs = torch.rand(layers, kvh, t_long, device=dev) * 0.05
    table_long = torch.randn(t_long, d, device=dev).to(torch.bfloat16)
    pos_long = torch.tensor([ctx_long], dtype=torch.int32, device=dev)
    partials = torch.zeros(ext.kv_attend_partials_floats(qh, d, 64), device=dev)

    def longest_step():
        for layer in range(layers):
            ext.kv_rope_append_attend_split(qkv, table_long, table_long, kc[layer], vc[layer], ks[layer], vs[layer],
                                            partials, pos_long, d ** -0.5, qh, 64)

    nbytes = 2 * kvh * (ctx_long + 1) * d + 2 * kvh * (ctx_long + 1) * 4
    us = round(_graph_time_us(torch, longest_step, reps=20) / layers, 2)
    out["kv_int8_rope_append_attention_ctx131000_per_layer"] = {
        "bytes": nbytes, "four_heads_matrix_core_64_splits_us": us, "GBps": round(nbytes / us / 1e3, 1),
        "frac_hbm": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)}
    del kc, vc, ks, vs, table_long
    # and for heads of 128 (the Llama-3-8B geometry), 5 layers = 350 MB
    layers, d = 5, 128
    kc = torch.randint(0, 100, (layers, kvh, t_max, d), device=dev).to(torch.int8)
    vc = torch.randint(0, 100, (layers, kvh, t_max, d), device=dev).to(torch.int8)
    ks = torch.rand(layers, kvh, t_max, device=dev) * 0.05
    vs = torch.rand(layers, kvh, t_max, device=dev) * 0.05
    qkv = torch.randn(1, (qh + 2 * kvh) * d, device=dev).to(torch.bfloat16)
    table = torch.randn(t_max, d, device=dev).to(torch.bfloat16)
    partials = torch.zeros(ext.kv_attend_partials_floats(qh, d, 32), device=dev)

    def long_step_128():
        for layer in range(layers):
            ext.kv_rope_append_attend_split(qkv, table, table, kc[layer], vc[layer], ks[layer], vs[layer], partials,
                                            pos, d ** -0.5, qh, 32)

    nbytes = 2 * kvh * (ctx + 1) * d + 2 * kvh * (ctx + 1) * 4
    us = round(_graph_time_us(torch, long_step_128, reps=20) / layers, 2)
    out["kv_int8_rope_append_attention_ctx32000_head_dim128_per_layer"] = {
        "bytes": nbytes, "four_heads_matrix_core_32_splits_us": us, "GBps": round(nbytes / us / 1e3, 1),
        "frac_hbm": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)}
    del kc, vc, ks, vs
    # the GEMV on Llama-3-8B's linears (M = 1): random codes, buffers rotated over > 600 MB so that
    # every launch streams from HBM; the launches of one rotation replayed as a HIP graph
    shapes_8b = []
    for name, n, k in (("q/o", 4096, 4096), ("k/v", 1024, 4096), ("gate/up", 14336, 4096),
                       ("down", 4096, 14336), ("lm_head", 128256, 4096)):
        x = torch.randn(1, k, device=dev).to(torch.bfloat16)
        for bits in (8, 4):
            nbytes = algorithmic_bytes(n, k, bits)
            copies = max(2, min(24, (600 << 20) // nbytes + 1))
            width = GROUP if bits == 8 else GROUP // 2
            qs = [torch.randint(0, 255, (n, k // GROUP, width), dtype=torch.uint8, device=dev) for _ in range(copies)]
            if bits == 8:
                qs = [q.view(torch.int8) for q in qs]
            sw = torch.rand(n, k // GROUP, device=dev) * 0.01
            outs = torch.empty(copies, 1, n, device=dev, dtype=torch.bfloat16)
            lib = _CAPI["lib"]
            sptr_of = lambda: ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

            def sweep():  # one launch per buffer copy, through the C ABI (no allocation: graph-safe)
                sp = sptr_of()
                for c in range(copies):
                    rc = lib.llmq_wq_gemv(x.data_ptr(), qs[c].data_ptr(), sw.data_ptr(), outs[c].data_ptr(),
                                          1, n, k // GROUP, GROUP, 0, bits, 2, sp)
                    if rc:
                        raise RuntimeError(lib.llmq_last_error().decode())

            us = _graph_time_us(torch, sweep, reps=5) / copies
            shapes_8b.append({"shape": name, "N": n, "K": k, "bits": bits, "bytes": nbytes, "us": round(us, 2),
                              "GBps": round(nbytes / us / 1e3, 1),
                              "frac_hbm": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)})
            del qs
    out["gemv_llama3_8b_shapes_graph_replay"] = shapes_8b
    # Mixture-of-Experts decode, OLMoE-1B-7B geometry (64 experts, top-8, hidden 2048, intermediate 1024,
    # int4): the two batched launches of one layer for one token; 16 layers' stacks rotated, as a graph
    from llmquant.quantizers import route_plan

    experts, top_k, hid, inter, layers = 64, 8, 2048, 1024, 16
    gu = [torch.randint(0, 255, (experts, 2 * inter, hid // GROUP, GROUP // 2), dtype=torch.uint8, device=dev)
          for _ in range(layers)]
    dn = [torch.randint(0, 255, (experts, hid, inter // GROUP, GROUP // 2), dtype=torch.uint8, device=dev)
          for _ in range(layers)]
    sgu = torch.rand(experts, 2 * inter, hid // GROUP, device=dev) * 0.01
    sdn = torch.rand(experts, hid, inter // GROUP, device=dev) * 0.01
    index = torch.randperm(experts, device=dev)[:top_k][None]
    _, plan = route_plan(index, experts, ext.wq_gemv_batched_max_rows())
    rows_h = torch.randn(top_k, hid, device=dev).to(torch.bfloat16)
    rows_i = torch.randn(top_k, inter, device=dev).to(torch.bfloat16)

    def moe_step():
        for layer in range(layers):
            ext.wq_gemv_batched(rows_h, gu[layer], sgu, *plan, 0)
            ext.wq_gemv_batched(rows_i, dn[layer], sdn, *plan, 0)

    us = _graph_time_us(torch, moe_step, reps=10) / layers
    nbytes = top_k * (2 * inter * hid // 2 + hid * inter // 2 + (2 * inter * hid // GROUP + hid * inter // GROUP) * 4)
    out["moe_batched_gemv_olmoe_int4_top8_per_layer"] = {
        "us": round(us, 2), "bytes": nbytes, "GBps": round(nbytes / us / 1e3, 1),
        "frac_hbm": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4), "launches": 2}
    # the whole experts block for one token (routing plan, both projections, weighted sum): the module's
    # four-launch forward against the operation-by-operation form of the reference's KernelQuantExperts
    from llmquant.core.scheme import QuantizationArgs, QuantizationScheme
    from llmquant.quantizers import KernelQuantExperts

    scheme = QuantizationScheme(weights=QuantizationArgs(4, "group", group_size=GROUP), input_activations=None)
    block = KernelQuantExperts(gu[0], sgu, dn[0], sdn, scheme, hid, inter, torch.nn.SiLU()).to(dev)
    hidden = torch.randn(1, hid, device=dev).to(torch.bfloat16)
    gates = torch.rand(1, top_k, device=dev).to(torch.bfloat16)
    fused_us = _graph_time_us(torch, lambda: [block(hidden, index, gates) for _ in range(layers)], reps=10) / layers
    plain_us = _graph_time_us(torch, lambda: [block._forward_unfused(hidden, index, gates) for _ in range(layers)],
                              reps=10) / layers
    out["moe_experts_block_one_token_olmoe_int4"] = {"us": round(fused_us, 2), "launches": 4,
                                                     "operation_by_operation_us": round(plain_us, 2)}
    del gu, dn, block
    # integer GEMM, Llama-3-8B MLP shapes
    gemm = []
    for n, k in ((14336, 4096), (4096, 14336)):
        # eleven copies of the 29 MB weight, one per launch in turn: no launch finds its weight in the
        # 256 MB Infinity Cache
        copies = (300 << 20) // (n * k // 2) + 1
        q4s = [torch.randint(0, 255, (n, k // GROUP, GROUP // 2), dtype=torch.uint8, device=dev) for _ in range(copies)]
        sw = torch.rand(n, k // GROUP, device=dev) * 0.01
        turn = [0]
        for m in (128, 512, 2048):
            x = torch.randn(m, k, device=dev).to(torch.bfloat16)
            a, sx = ext.quant_group_codes(x, 8, GROUP, False)

            def one():
                turn[0] += 1
                return ext.wq_gemm_a8(a, sx, q4s[turn[0] % copies], sw)

            def fast():
                turn[0] += 1
                return ext.wq_gemm_a8(a, sx, q4s[turn[0] % copies], sw, None, 0, torch.bfloat16, False)

            sx_token = sx[:, :1].contiguous()   # (timing only: what one scale per token costs to apply)

            def fast_token():
                turn[0] += 1
                return ext.wq_gemm_a8(a, sx_token, q4s[turn[0] % copies], sw, None, 0, torch.bfloat16, False)

            us_natural = _event_time_us(torch, one, reps=2 * copies)
            us_f = _event_time_us(torch, fast, reps=2 * copies)
            us_t = _event_time_us(torch, fast_token, reps=2 * copies)
            us_q = _event_time_us(torch, lambda: ext.quant_group_codes(x, 8, GROUP, False), reps=10)
            # what KernelQuantLinear calls for the shape: where the exact form runs its group-parallel kernel, the
            # quantizer writes the codes in that kernel's operand order (same codes, same result bit for bit)
            operand_order = bool(ext.wq_gemm_a8_takes_groups(m, n, k // GROUP))
            us = us_natural
            if operand_order:
                a_tiled, sx_tiled = ext.quant_act_codes_tiled(x, 4)

                def tiled_call():
                    turn[0] += 1
                    return ext.wq_gemm_a8_tiled(a_tiled, sx_tiled, m, q4s[turn[0] % copies], sw)

                us = _event_time_us(torch, tiled_call, reps=2 * copies)
                us_q = _event_time_us(torch, lambda: ext.quant_act_codes_tiled(x, 4), reps=10)
            gemm.append({"M": m, "N": n, "K": k, "weights": "int4", "gemm_us": round(us, 1),
                         "codes": "operand order (llmq_wq_gemm_a8_tiled)" if operand_order else "[M, K] (llmq_wq_gemm_a8)",
                         "gemm_us_on_codes_in_natural_order": round(us_natural, 1),
                         "act_quant_us": round(us_q, 1), "TOPS": round(2 * m * n * k / us / 1e6, 1),
                         "frac_int8_mfma_peak": round(2 * m * n * k / us / 1e6 / 5000.0, 4),
                         "fast_form_us": round(us_f, 1), "fast_form_TOPS": round(2 * m * n * k / us_f / 1e6, 1),
                         "fast_form_frac_int8_mfma_peak": round(2 * m * n * k / us_f / 1e6 / 5000.0, 4),
                         "fast_form_one_scale_per_token_us": round(us_t, 1),
                         "fast_form_one_scale_per_token_TOPS": round(2 * m * n * k / us_t / 1e6, 1),
                         "weights_rotated_over_bytes": copies * (n * k // 2)})
        del q4s
    out["w4a8_gemm"] = gemm
    # prompt-sized bf16 (one row: fp16) activations: the tiled fused GEMM (no dense weight) against the branch it
    # replaces (one-pass dequantize + the BLAS library's matmul), weights rotated the same way; `routed_to` is what
    # KernelQuantLinear.forward picks for the shape (tiled_gemm_pays: the estimated times of the two branches)
    from llmquant.quantizers.kernel import tiled_gemm_pays

    tiled = []
    for m, n, k, bits, dtype in ((512, 16384, 2048, 4, torch.bfloat16), (512, 2048, 8192, 4, torch.bfloat16),
                                 (512, 3072, 2048, 8, torch.bfloat16), (512, 3072, 2048, 4, torch.bfloat16),
                                 (192, 3072, 2048, 8, torch.bfloat16), (128, 14336, 4096, 4, torch.bfloat16),
                                 (512, 14336, 4096, 4, torch.bfloat16), (512, 14336, 4096, 4, torch.float16),
                                 (640, 14336, 4096, 4, torch.bfloat16), (1024, 2048, 8192, 4, torch.bfloat16),
                                 (2048, 14336, 4096, 4, torch.bfloat16), (2048, 4096, 14336, 4, torch.bfloat16)):
        copies = min(24, (300 << 20) // (n * k * bits // 8) + 1)
        width = GROUP if bits == 8 else GROUP // 2
        qs = [torch.randint(0, 255, (n, k // GROUP, width), dtype=torch.uint8, device=dev) for _ in range(copies)]
        if bits == 8:
            qs = [q.view(torch.int8) for q in qs]
        sw = torch.rand(n, k // GROUP, device=dev) * 0.01 + 1e-3
        x = torch.randn(m, k, device=dev).to(dtype)
        turn = [0]

        def fused_call():
            turn[0] += 1
            return ext.wq_gemm_a16_tile(x, qs[turn[0] % copies], sw, 0)

        def dense_call():
            turn[0] += 1
            return ext.wq_dense_linear(x, qs[turn[0] % copies], sw, 0, 0)

        us_f = _event_time_us(torch, fused_call, reps=2 * copies)
        us_d = _event_time_us(torch, dense_call, reps=2 * copies)
        tiled.append({"M": m, "N": n, "K": k, "weights": f"int{bits}",
                      "activations": "bf16" if dtype == torch.bfloat16 else "fp16", "us": round(us_f, 1),
                      "TFLOPs": round(2 * m * n * k / us_f / 1e6, 1),
                      "frac_bf16_mfma_peak": round(2 * m * n * k / us_f / 1e6 / 2500.0, 4),
                      "dequant_plus_matmul_us": round(us_d, 1),
                      "routed_to": "tiled" if tiled_gemm_pays(m, n, k // GROUP, bits) else "dequant_plus_matmul"})
        del qs
    out["w4a16_tiled_gemm_prompt_m"] = tiled
    # a few dozen rows of a 16-bit activation: the fused GEMM (codes straight from HBM to the matrix cores)
    # against the dense branch it replaces (dequantize the weight, then a dense matmul), Llama-3-8B MLP
    # shapes, int4, weights rotated over > 600 MB, one rotation replayed as a graph
    lib = _CAPI["lib"]
    fused = []
    for n, k in ((14336, 4096), (4096, 14336)):
        nbytes_w = n * k // 2 + n * (k // GROUP) * 4
        copies = (600 << 20) // nbytes_w + 1
        qs = [torch.randint(0, 255, (n, k // GROUP, GROUP // 2), dtype=torch.uint8, device=dev) for _ in range(copies)]
        sw = torch.rand(n, k // GROUP, device=dev) * 0.01
        for m in (8, 16, 32, 64):
            x = torch.randn(m, k, device=dev).to(torch.bfloat16)
            y = torch.empty(m, n, device=dev, dtype=torch.bfloat16)
            dense = torch.empty(n, k, device=dev, dtype=torch.bfloat16)

            def fused_sweep():
                sp = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
                for c in range(copies):
                    rc = lib.llmq_wq_gemm_a16(x.data_ptr(), qs[c].data_ptr(), sw.data_ptr(), y.data_ptr(), m, n,
                                              k // GROUP, GROUP, 0, 4, 2, sp)
                    if rc:
                        raise RuntimeError(lib.llmq_last_error().decode())

            def dense_sweep():
                sp = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
                for c in range(copies):
                    rc = lib.llmq_dequant_weight(qs[c].data_ptr(), sw.data_ptr(), dense.data_ptr(), n, k // GROUP,
                                                 GROUP, GROUP, 0, 4, 2, sp)
                    if rc:
                        raise RuntimeError(lib.llmq_last_error().decode())
                    torch.matmul(x, dense.T, out=y)

            need = lib.llmq_wq_gemm_a16_workspace_bytes(m, n, k // GROUP)
            scratch = torch.empty(max(need // 4, 4), device=dev)

            def split_sweep():  # the reduction axis split across workgroups: two launches, flat in M
                sp = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
                for c in range(copies):
                    rc = lib.llmq_wq_gemm_a16_split(x.data_ptr(), qs[c].data_ptr(), sw.data_ptr(), y.data_ptr(),
                                                    scratch.data_ptr(), need, m, n, k // GROUP, GROUP, 0, 4, 2, sp)
                    if rc:
                        raise RuntimeError(lib.llmq_last_error().decode())

            us_whole = _graph_time_us(torch, fused_sweep, reps=5) / copies
            us_split = _graph_time_us(torch, split_sweep, reps=5) / copies
            us_dense = _graph_time_us(torch, dense_sweep, reps=5) / copies
            us = us_whole  # KernelQuantLinear's choice (fused_gemm_splits: the whole-rows form everywhere)
            nbytes = nbytes_w + m * k * 2 + m * n * 2
            fused.append({"M": m, "N": n, "K": k, "weights": "int4", "us": round(us, 2),
                          "whole_rows_form_us": round(us_whole, 2), "split_form_us": round(us_split, 2),
                          "dequant_plus_matmul_us": round(us_dense, 2), "bytes": nbytes,
                          "GBps": round(nbytes / us / 1e3, 1), "frac_hbm": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)})
        del qs
    out["w4a16_fused_gemm_small_m"] = fused

    # The prompt's causal grouped-query attention (Llama-3.2-1B geometry: 32 query / 8 kv heads of 64; and the
    # 8B head size), the package's kernel beside torch's scaled_dot_product_attention + the copy that brings its
    # output to [tokens, heads * head_dim]. Flops: 4 * tokens^2 / 2 * heads * head_dim.
    attention = []
    for tokens, d in ((128, 64), (512, 64), (2048, 64), (512, 128)):
        qh, kvh = 32, 8
        q = torch.randn(tokens, qh, d, device=dev).to(torch.bfloat16)
        kk = torch.randn(kvh, tokens, d, device=dev).to(torch.bfloat16)
        vv = torch.randn(kvh, tokens, d, device=dev).to(torch.bfloat16)

        def ours():
            for _ in range(10):
                ext.prefill_attention(q, kk, vv, d ** -0.5)

        def library():
            for _ in range(10):
                ctx = torch.nn.functional.scaled_dot_product_attention(q.transpose(0, 1)[None], kk[None], vv[None],
                                                                       is_causal=True, scale=d ** -0.5, enable_gqa=True)
                ctx[0].transpose(0, 1).reshape(tokens, -1)

        us = _graph_time_us(torch, ours, reps=10) / 10
        us_lib = _graph_time_us(torch, library, reps=10) / 10
        flops = 2 * tokens * tokens * qh * d
        attention.append({"tokens": tokens, "q_heads": qh, "kv_heads": kvh, "head_dim": d, "us": round(us, 2),
                          "TFLOPs": round(flops / us / 1e6, 1), "torch_sdpa_us": round(us_lib, 2)})
    out["prompt_attention_bf16"] = attention
    return out


def decode_leg(torch, arch="llama3.2-1b"):
    """The end-to-end decode case: random-init Llama-3.2-1B architecture, attention int8 / MLP int4 /
    lm_head int8 / int8 KV cache, 512-token prompt, 256 greedy tokens, batch 1. TTFT = median
    time of generating 1 token; decode tok/s = (n - 1) / (median time of n tokens - TTFT), the
    reference's definition (llmquant/eval/evaluate.py:209-218). Both sides replay a captured step.
    arch "llama3-8b": the same on the Llama-3-8B architecture (the other model of the layer-shape target; not
    part of the default run), 128 new tokens."""
    import time

    from transformers import LlamaConfig, LlamaForCausalLM

    from llmquant import QuantConfig, oneshot

    torch.manual_seed(0)
    shape = {"llama3.2-1b": dict(hidden_size=2048, intermediate_size=8192, num_hidden_layers=16, head_dim=64),
             "llama3-8b": dict(hidden_size=4096, intermediate_size=14336, num_hidden_layers=32, head_dim=128)}[arch]
    cfg = LlamaConfig(num_attention_heads=32, num_key_value_heads=8, vocab_size=128256, rms_norm_eps=1e-5,
                      rope_parameters={"rope_type": "default", "rope_theta": 500000.0},
                      tie_word_embeddings=False, max_position_embeddings=4096, **shape)
    with torch.device("cuda:0" if arch == "llama3-8b" else "cpu"):   # (16 GB of bf16: built where it will live)
        model = LlamaForCausalLM(cfg)
    for p in model.parameters():
        if p.dim() > 1:
            torch.nn.init.normal_(p, 0, 0.02)
    model = model.to(torch.bfloat16).to("cuda:0").eval()
    prompt, new = 512, (256 if arch == "llama3.2-1b" else 128)
    from llmquant.eval import latency_row, measure_latency, reconcile

    def measure(kv_bits):
        lat = measure_latency(model, None, prompt_tokens=prompt, new_tokens=new, iters=3, use_cuda_graph=True,
                              kv_bits=kv_bits)
        return lat, {"ttft_ms": round(lat["ttft_ms"], 2), "decode_tok_s": round(lat["decode_tps"], 1)}

    res = {"architecture": arch, "prompt_tokens": prompt, "new_tokens": new, "hip_graph": True,
           "paths": {"bf16_fused_runtime": "the bf16 model through the same five-launch step as the quantized one: "
                                           "LlamaDenseFusedRuntime (llmq_dense_gemv_fused over the bf16 weights, "
                                           "unquantized bf16 KV cache), one captured step, kept between calls",
                     "bf16_hf_walk": "HF LlamaForCausalLM module walk over a StaticCache, one captured step, kept "
                                     "between calls (hf_static_cache_graph)",
                     "kernel": "LlamaFusedRuntime: five launches per layer, integer KV cache, one captured step, "
                               "kept between calls (fused_runtime_graph)",
                     "kernel_kv_bf16_fused_runtime": "the kernel-mode model under the same fused runtime with its "
                                                     "cache left at bf16 (the kv_cache=bf16 ablation)",
                     "kernel_kv_bf16_hf_walk": "the kernel-mode model under the HF module walk over a StaticCache "
                                               "(the reference's arrangement for a weight-only recipe)"},
           "note": "speedup_vs_bf16 is kernel / bf16_fused_runtime: both sides run the same five-launch step under "
                   "graph replay, so it prices the quantization alone. speedup_vs_bf16_hf_walk compares against the "
                   "HF module walk (about 40 launches per layer) and is mostly the runtime."}
    from llmquant.eval import deployed_cost

    lat_bf16_walk, res["bf16_hf_walk"] = measure(None)
    lat_bf16, res["bf16_fused_runtime"] = measure(16)
    cost_bf16 = deployed_cost(model, None)
    from llmquant.runtime import drop_kept

    drop_kept(model)
    recipe = QuantConfig(attn_weight="int8", mlp_weight="int4", head_weight="int8", kv_cache="int8")
    oneshot(model, recipe.to_modifier("kernel"))
    torch.cuda.empty_cache()
    cost_kernel, cost_abl = deployed_cost(model, 8), deployed_cost(model, None)
    lat_kernel, res["kernel"] = measure(8)
    # ablation row of the verification plan: the selected recipe with the KV cache back at bf16, under the same
    # fused runtime, and under the HF walk as the reference arranges it
    lat_abl, res["kernel_kv_bf16_fused_runtime"] = measure(16)
    lat_abl_walk, res["kernel_kv_bf16_hf_walk"] = measure(None)
    res["config"] = recipe.describe()
    res["speedup_vs_bf16"] = round(res["kernel"]["decode_tok_s"] / res["bf16_fused_runtime"]["decode_tok_s"], 3)
    res["speedup_vs_bf16_hf_walk"] = round(res["kernel"]["decode_tok_s"] / res["bf16_hf_walk"]["decode_tok_s"], 3)
    res["hf_walk_speedup_of_the_weights_alone"] = round(res["kernel_kv_bf16_hf_walk"]["decode_tok_s"]
                                                        / res["bf16_hf_walk"]["decode_tok_s"], 3)
    # the same runs as rows of the reference's report format (eval/run.py, eval/verify.py): the plan's three rows
    # all under the fused runtime, the two HF-walk runs beside them
    from dataclasses import replace

    from llmquant.eval import verification_plan

    plan = verification_plan(recipe)
    measured = {"bf16 baseline": (None, "fused_runtime_graph", lat_bf16, cost_bf16),
                "selected": (recipe, "fused_runtime_graph", lat_kernel, cost_kernel),
                "selected, kv_cache=bf16": (replace(recipe, kv_cache="bf16"), "fused_runtime_graph", lat_abl, cost_abl)}
    rows = [dict(latency_row(*measured[label][:3], cost=measured[label][3]), verify_label=label)
            for label, _ in plan if label in measured]
    res["verify"] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in reconcile(rows).items()}
    rows.append(dict(latency_row(None, "hf_static_cache_graph", lat_bf16_walk, cost=cost_bf16),
                     verify_label="bf16 baseline, HF module walk"))
    rows.append(dict(latency_row(replace(recipe, kv_cache="bf16"), "hf_static_cache_graph", lat_abl_walk, cost=cost_abl),
                     verify_label="selected, kv_cache=bf16, HF module walk"))
    res["verify_rows"] = [{k: (round(v, 4) if isinstance(v, float) else v) for k, v in row.items()} for row in rows]
    del model
    torch.cuda.empty_cache()
    if arch == "llama3.2-1b":
        res["token_identity_first_64"] = token_identity(torch, cfg, recipe, prompt)
    return res


def token_identity(torch, cfg, recipe, prompt):
    """The first 64 greedy tokens, free-running on both sides: graphed_generate (the fused step under graph
    replay, what the tok/s above is measured on) against the same weights in the package's real mode under HF
    transformers with the PyTorch-side quantized cache -- on the architecture built in float32 (where the two
    differ by fp32 summation order only and the streams must be identical) and in bfloat16 (where a random-init
    model's own logits tie and two correct implementations part at the first near-tie)."""
    import copy

    from transformers import LlamaForCausalLM

    from llmquant import oneshot
    from llmquant.quantizers import make_cache_factory
    from llmquant.runtime import graphed_generate

    out = {}
    ids = torch.randint(0, cfg.vocab_size, (1, prompt), generator=torch.Generator().manual_seed(1)).to("cuda:0")
    for tag, dtype in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
        torch.manual_seed(0)
        model = LlamaForCausalLM(cfg)
        for p in model.parameters():
            if p.dim() > 1:
                torch.nn.init.normal_(p, 0, 0.02)
        model = model.to(dtype).to("cuda:0").eval()
        real = oneshot(copy.deepcopy(model), recipe.to_modifier("real"))
        kernel = oneshot(model, recipe.to_modifier("kernel"))
        cache = make_cache_factory(8)()
        want, gaps = [], []
        with torch.no_grad():
            logits = real(ids, past_key_values=cache, use_cache=True).logits[0, -1].float()
            for _ in range(64):
                top2 = logits.topk(2).values
                gaps.append((top2[0] - top2[1]).item())
                tok = logits.argmax().reshape(1, 1)
                want.append(tok.item())
                logits = real(tok, past_key_values=cache, use_cache=True).logits[0, -1].float()
        got = graphed_generate(kernel, ids, 64, kv_bits=8)[0, prompt:].tolist()
        prefix = next((i for i, (a, b) in enumerate(zip(got, want)) if a != b), 64)
        out[tag] = {"identical_prefix": prefix, "positions_equal": sum(a == b for a, b in zip(got, want)),
                    "oracle_min_top2_gap": round(min(gaps), 6),
                    "oracle_top2_gap_where_the_streams_part": round(gaps[prefix], 6) if prefix < 64 else None}
        del model, real, kernel, cache
        torch.cuda.empty_cache()
    return out


def prefill_leg(torch, prompt=512):
    """The prompt pass of config 5 by itself: twelve prefills of `prompt` tokens through the kernel runtime on the
    random-init Llama-3.2-1B architecture (attention int8 / MLP int4 / lm_head int8 / int8 KV), wall time
    and HIP events per call. The run to profile for what a time-to-first-token is made of."""
    import time

    from transformers import LlamaConfig, LlamaForCausalLM

    from llmquant import QuantConfig, oneshot
    from llmquant.runtime import kernel_runtime

    torch.manual_seed(0)
    cfg = LlamaConfig(hidden_size=2048, intermediate_size=8192, num_hidden_layers=16, num_attention_heads=32,
                      num_key_value_heads=8, head_dim=64, vocab_size=128256, rms_norm_eps=1e-5,
                      rope_parameters={"rope_type": "default", "rope_theta": 500000.0},
                      tie_word_embeddings=False, max_position_embeddings=4096)
    model = LlamaForCausalLM(cfg).to(torch.bfloat16).to("cuda:0").eval()
    oneshot(model, QuantConfig(attn_weight="int8", mlp_weight="int4", head_weight="int8",
                               kv_cache="int8").to_modifier("kernel"))
    ids = torch.randint(0, 128256, (1, prompt), generator=torch.Generator().manual_seed(1)).to("cuda:0")
    wall, gpu, host = [], [], []
    with torch.no_grad():
        runtime = kernel_runtime(model, prompt + 2, 8)
        for rep in range(15):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            a.record()
            runtime.prefill(ids)
            t1 = time.perf_counter()   # every launch of the pass is queued (nothing in it waits for the GPU)
            b.record()
            torch.cuda.synchronize()
            if rep >= 3:
                wall.append((time.perf_counter() - t0) * 1e3)
                gpu.append(a.elapsed_time(b))
                host.append((t1 - t0) * 1e3)
    wall.sort(), gpu.sort(), host.sort()
    return {"prompt_tokens": prompt, "calls": len(wall), "runtime": type(runtime).__name__,
            "median_wall_ms": round(wall[len(wall) // 2], 3), "median_events_ms": round(gpu[len(gpu) // 2], 3),
            "median_host_queueing_ms": round(host[len(host) // 2], 3)}


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
    result = {"value": round(step_bytes * steps / elapsed / 1e9, 2), "unit": "GB/s",
              "cores": int(olib.llmq_oracle_threads()), "kind": "port",
              "sample": f"{steps} full steps of the same sweep (same operands) in {elapsed:.1f} s, "
                        f"OpenMP over output rows",
              "cpu": model, "os_cpu_count": os.cpu_count()}
    result["fake"] = cpu_fake_sweep(torch, cases, min(6.0, budget_s))
    result["w4a8_gemm"] = cpu_w4a8_gemm(torch, olib)
    result["decode"] = cpu_decode(torch)
    return result


def cpu_fake_sweep(torch, cases, budget_s: float):
    """The reference's fake path (llmquant/quantizers/fake.py:18-36: weights quantize-dequantized once and kept
    in bf16, then F.linear) on the host cores, on the same sweep and the same operands: the package's
    FakeQuantLinear over the dequantized weight of every shape, torch CPU, all threads torch is given. `value` is
    in the unit of the GPU figure (the sweep's algorithmic bytes in their quantized form per second); what the
    host actually streams is the bf16 weight, reported beside it."""
    from llmquant.core.scheme import QuantizationArgs, QuantizationScheme
    from llmquant.quantizers import FakeQuantLinear

    threads = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(threads)
    layers, bf16_bytes = [], 0
    for case in cases:
        q, s = case["bufs"][0]
        from llmquant.packing.packing import unpack_int4

        codes = unpack_int4(q) if case["bits"] == 4 else q
        weight = (codes.float() * s[:, :, None]).reshape(case["n"], case["k"]).to(torch.bfloat16).cpu()
        scheme = QuantizationScheme(weights=QuantizationArgs(case["bits"], "group", group_size=GROUP),
                                    input_activations=None)
        layers.append((FakeQuantLinear(weight, None, scheme), case["x"].cpu()))
        bf16_bytes += weight.numel() * 2
    step_bytes = sum(c["bytes"] for c in cases)

    def one_step():
        with torch.no_grad():
            for layer, x in layers:
                layer(x)

    one_step()
    t0 = time.perf_counter()
    steps = 0
    while time.perf_counter() - t0 < budget_s:
        one_step()
        steps += 1
    elapsed = time.perf_counter() - t0
    return {"value": round(step_bytes * steps / elapsed / 1e9, 2), "unit": "GB/s", "cores": threads, "kind": "port",
            "bf16_weight_GBps": round(bf16_bytes * steps / elapsed / 1e9, 2),
            "sample": f"{steps} full steps of the same sweep through FakeQuantLinear (dequantized bf16 weights + "
                      f"F.linear, torch CPU) in {elapsed:.1f} s"}


def cpu_w4a8_gemm(torch, olib):
    """The integer prefill GEMM (int8 activations per token x group, int4 weights) through the C oracle's
    real-mode arithmetic on the host cores: a slice of the 14336 x 4096 Llama-3-8B case small enough to
    finish in seconds (the cost is linear in M and N, so the rate carries over)."""
    import numpy as np

    m, n, k = 64, 2048, 4096
    rng = np.random.default_rng(0)
    a = rng.integers(-127, 128, (m, k), dtype=np.int8)
    sx = (rng.random((m, k // GROUP), dtype=np.float32) * 0.05 + 1e-3)
    qw = rng.integers(0, 256, (n, k // GROUP, GROUP // 2), dtype=np.uint8)
    ws = (rng.random((n, k // GROUP), dtype=np.float32) * 0.01 + 1e-3)
    out = np.empty((m, n), dtype=np.float32)
    ptr = lambda arr: arr.ctypes.data_as(ctypes.c_void_p)
    olib.llmq_oracle_real_gemm_a8.restype = None
    call = lambda: olib.llmq_oracle_real_gemm_a8(ptr(a), ptr(sx), ptr(qw), ptr(ws), ptr(out), m, n, k // GROUP,
                                                 GROUP, 0, 1)
    call()
    t0 = time.perf_counter()
    reps = 0
    while time.perf_counter() - t0 < 4.0:
        call()
        reps += 1
    elapsed = time.perf_counter() - t0
    return {"value": round(2.0 * m * n * k * reps / elapsed / 1e12, 4), "unit": "TOPS",
            "cores": int(olib.llmq_oracle_threads()), "kind": "port",
            "sample": f"{reps} x (M={m}, N={n}, K={k}) int4 weights, a {m}x{n} slice of the 14336 x 4096 case, "
                      f"{elapsed:.1f} s"}


def cpu_decode(torch):
    """The end-to-end decode case shortened for the host: the same random-init Llama-3.2-1B architecture and
    recipe in the package's real mode (integer weights, fp32 matmul per group: the reference's CPU-capable
    path) with the PyTorch-side quantized cache, 32 prompt tokens and 8 greedy tokens on the host cores."""
    from transformers import LlamaConfig, LlamaForCausalLM

    from llmquant import QuantConfig, oneshot
    from llmquant.quantizers import make_cache_factory

    threads = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(threads)
    torch.manual_seed(0)
    cfg = LlamaConfig(hidden_size=2048, intermediate_size=8192, num_hidden_layers=16, num_attention_heads=32,
                      num_key_value_heads=8, head_dim=64, vocab_size=128256, rms_norm_eps=1e-5,
                      rope_parameters={"rope_type": "default", "rope_theta": 500000.0},
                      tie_word_embeddings=False, max_position_embeddings=4096)
    # (built and quantized on the GPU, which takes seconds, then moved to the host: only the timed part runs there)
    with torch.device("cuda:0"):
        model = LlamaForCausalLM(cfg).to(torch.bfloat16).eval()
    recipe = QuantConfig(attn_weight="int8", mlp_weight="int4", head_weight="int8", kv_cache="int8")
    oneshot(model, recipe.to_modifier("real"))
    model = model.cpu()
    torch.cuda.empty_cache()
    prompt, new = 32, 8
    ids = torch.randint(0, 128256, (1, prompt), generator=torch.Generator().manual_seed(1))
    cache = make_cache_factory(8)()
    with torch.no_grad():
        t0 = time.perf_counter()
        logits = model(ids, past_key_values=cache, use_cache=True).logits[:, -1]
        ttft = time.perf_counter() - t0
        tok = logits.argmax(-1, keepdim=True)
        t1 = time.perf_counter()
        for _ in range(new - 1):
            tok = model(tok, past_key_values=cache, use_cache=True).logits[:, -1].argmax(-1, keepdim=True)
        decode = time.perf_counter() - t1
    return {"value": round((new - 1) / decode, 3), "unit": "tok/s", "cores": threads, "kind": "port",
            "ttft_ms": round(ttft * 1e3, 1),
            "sample": f"real mode on the host, prompt {prompt} tokens, {new} greedy tokens ({decode:.1f} s of decode)"}


if __name__ == "__main__":
    main()
