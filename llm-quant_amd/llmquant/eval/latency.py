"""Prefill TTFT and steady-state decode throughput, by the reference's definition
(llmquant/eval/evaluate.py:167-223), and the result row a run reports (llmquant/eval/run.py:108-159).

TTFT is the median time of generating one token; decode tokens/s is (n - 1) divided by the median
time of generating n tokens minus the TTFT, so the two regimes (compute-bound prefill,
bandwidth-bound decode) are reported apart.
"""

from __future__ import annotations

import time

import torch

from llmquant.core.config import QuantConfig, normalize_dtype


@torch.no_grad()
def measure_latency(model, tokenizer=None, prompt_tokens: int = 512, new_tokens: int = 64, iters: int = 3,
                    cache_factory=None, use_cuda_graph: bool = False, kv_bits=None, seed: int = 1):
    """Same keys as the reference's measure_latency. `tokenizer` may be None (vocab size and pad
    token then come from model.config; there is no checkpoint offline). `kv_bits` selects the
    integer-KV kernel runtime for graphed runs of a kernel-mode model; without it graphed runs
    take the HF static-cache path and ungraphed runs call model.generate, as the reference does."""
    device = next(model.parameters()).device
    vocab = tokenizer.vocab_size if tokenizer is not None else model.config.vocab_size
    pad_id = tokenizer.eos_token_id if tokenizer is not None else 0
    gen = torch.Generator().manual_seed(seed)
    ids = torch.randint(0, vocab, (1, prompt_tokens), generator=gen).to(device)
    inputs = {"input_ids": ids, "attention_mask": torch.ones_like(ids)}

    graphed = False
    if use_cuda_graph:
        from llmquant.runtime import can_graph, graphed_generate

        graphed = kv_bits is not None or can_graph(model, cache_factory)

    def timed(n):
        torch.cuda.synchronize()
        start = time.perf_counter()
        if graphed:
            graphed_generate(model, ids, n, kv_bits=kv_bits)
        else:
            model.generate(**inputs, max_new_tokens=n, min_new_tokens=n, do_sample=False, pad_token_id=pad_id,
                           **({"past_key_values": cache_factory()} if cache_factory else {}))
        torch.cuda.synchronize()
        return time.perf_counter() - start

    timed(min(4, new_tokens))  # warm-up
    torch.cuda.reset_peak_memory_stats(device)
    first = sorted(timed(1) for _ in range(iters))[iters // 2]
    full = sorted(timed(new_tokens) for _ in range(iters))[iters // 2]
    return {
        "ttft_ms": first * 1e3,
        "decode_tps": (new_tokens - 1) / max(full - first, 1e-9),
        "cuda_graph": graphed,
        "peak_vram_gb": torch.cuda.max_memory_allocated(device) / 1024 ** 3,
        "latency_prompt_tokens": prompt_tokens,
        "latency_new_tokens": new_tokens,
    }


def latency_row(quant: QuantConfig | None, mode: str, latency: dict, eval_sec: float | None = None,
                cost: dict | None = None) -> dict:
    """The row run_one() writes for one configuration (llmquant/eval/run.py:108-159) without the accuracy
    columns: the recipe's axes, the cost columns when `cost` (llmquant.eval.deployed_cost) is given, the
    timings, and which path produced them (`latency_mode`). quant None = the bf16 baseline."""
    quantize = quant is not None
    q = quant or QuantConfig()
    row = {
        "name": q.describe() if quantize else "bf16",
        "quantize": quantize,
        "attn_weight": normalize_dtype(q.attn_weight),
        "mlp_weight": normalize_dtype(q.mlp_weight),
        "head_weight": normalize_dtype(q.head_weight),
        "activation": normalize_dtype(q.activation),
        "kv_cache": normalize_dtype(q.kv_cache),
        "group_size": q.group_size,
    }
    if cost is not None:
        from llmquant.eval.cost import cost_columns

        row.update(cost_columns(cost))
    row.update(latency)
    row["latency_mode"] = mode
    if eval_sec is not None:
        row["eval_sec"] = eval_sec
    return row
