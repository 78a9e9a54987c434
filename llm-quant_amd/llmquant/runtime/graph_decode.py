"""Replaying a captured decode step (API of llmquant/runtime/graph_decode.py).

Two decoders share one interface (prefill / capture / step / logits / max_len):

  GraphedDecoder    any HF causal LM over a transformers StaticCache, the arrangement the
                    reference measures bf16 and weight-only runs with: eager prefill, warmup
                    on a side stream, one captured step, replay
  KernelDecoder     the kernel path with the integer KV cache (LlamaKernelRuntime): the case
                    the reference cannot graph, because its quantized cache is a growing
                    DynamicCache (graph_decode.py:40-43)

`graphed_generate` picks between them; both are used for the bf16-vs-quantized comparison so
neither side is credited with the graph alone.
"""

from __future__ import annotations

import torch

from llmquant.runtime.llama_decode import WARMUP_CALLS, LlamaKernelRuntime
from llmquant.runtime.llama_fused import LlamaDenseFusedRuntime, LlamaFusedRuntime

__all__ = ["GraphedDecoder", "KernelDecoder", "WARMUP_CALLS", "can_graph", "drop_kept", "graphed_generate",
           "kept_graphed_decoder", "kept_kernel_runtime", "kernel_runtime"]


def _on_gpu(model) -> bool:
    if not torch.cuda.is_available():
        return False
    first = next(model.parameters(), None)
    return first is not None and first.device.type == "cuda"


def can_graph(model, cache_factory=None) -> bool:
    """Whether a graphed decode is possible for this model and cache choice.

    A PyTorch-side quantized cache (FakeQuantCache factory) still cannot be captured; the
    kernel cache can, and is requested with `kv_bits` on graphed_generate instead of a factory.
    """
    if cache_factory is not None:
        return False
    return _on_gpu(model)


class GraphedDecoder:
    """One captured HF decode step over a StaticCache sized exactly to the run (attention
    costs the allocated length, and warmup/capture calls consume slots that are rewound)."""

    def __init__(self, model, prompt_tokens: int, new_tokens: int):
        from transformers import StaticCache

        self.model = model
        self.device = next(model.parameters()).device
        self.max_len = prompt_tokens + new_tokens + WARMUP_CALLS + 1
        self.cache = StaticCache(config=model.config, max_batch_size=1, max_cache_len=self.max_len,
                                 device=self.device, dtype=next(model.parameters()).dtype)
        self.token = torch.zeros(1, 1, dtype=torch.long, device=self.device)
        self.position = torch.zeros(1, dtype=torch.long, device=self.device)
        self.graph = None
        self.logits = None

    def _forward_token(self):
        return self.model(self.token, past_key_values=self.cache, use_cache=True,
                          position_ids=self.position.unsqueeze(0))

    @torch.no_grad()
    def prefill(self, input_ids):
        out = self.model(input_ids, past_key_values=self.cache, use_cache=True)
        return out.logits[:, -1:].argmax(-1)

    def _rewind(self, to: int):
        for layer in self.cache.layers:
            cursor = getattr(layer, "cumulative_length", None)
            if isinstance(cursor, torch.Tensor):
                cursor.fill_(to)

    @torch.no_grad()
    def capture(self, position: int):
        self.position.fill_(position)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(WARMUP_CALLS):
                self._forward_token()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            out = self._forward_token()
        self.logits = out.logits
        self._rewind(position)

    @torch.no_grad()
    def step(self, token, position: int):
        self.token.copy_(token.reshape(1, 1))
        self.position.fill_(position)
        self.graph.replay()
        return self.logits[:, -1:].argmax(-1)


def kernel_runtime(model, max_len: int, kv_bits: int = 8):
    """The fastest runtime the model qualifies for: the five-launches-per-layer fused step when
    every Linear is a weight-only kernel-mode module, else the operation-by-operation walk."""
    if kv_bits == 16:
        # an unquantized cache: the 16-bit baseline through the same fused step (plain nn.Linear modules), or
        # a kernel-mode model with its cache left at the model's dtype (the kv_cache=bf16 ablation)
        try:
            return LlamaDenseFusedRuntime(model, max_len, 16)
        except ValueError:
            return LlamaFusedRuntime(model, max_len, 16)
    try:
        return LlamaFusedRuntime(model, max_len, kv_bits)
    except ValueError:
        return LlamaKernelRuntime(model, max_len, kv_bits)


_KEPT_RUNTIMES = 4


class _Kept(dict):
    """What is kept on a model between generate calls (runtimes, captured graphs, the walked module tree). It
    belongs to that model object only: a deep copy or a pickle of the model carries an empty one (a captured
    graph can be neither copied nor pickled, and a copy's parameters live elsewhere anyway)."""

    def __deepcopy__(self, memo):
        return _Kept()

    def __reduce__(self):
        return (_Kept, ())


def _module_tree(model):
    """Every (parent, name, child) edge of the module tree and every place a tensor hangs in it (the
    `_parameters` / `_buffers` dict of a module and the name in it)."""
    edges, slots = [], []
    for parent in model.modules():
        for name, child in parent._modules.items():
            if child is not None:
                edges.append((parent, name, child))
        for holder in (parent._parameters, parent._buffers):
            for name, tensor in holder.items():
                if tensor is not None:
                    slots.append((holder, name))
    return _Kept(edges=edges, slots=slots)


def _weights_key(model):
    """Identity of everything a captured step has baked in: address, version and dtype of every parameter
    and buffer of the model: the quantized codes and scales, and also the embedding table, the norm weights
    and the rotary frequencies, whose addresses (or the tables computed from them) a captured step reads. A
    re-quantized or moved model, resize_token_embeddings, a norm weight replaced by a new Parameter, a
    load_state_dict(assign=True) or an in-place write all change it. The walk over the module tree is done
    once and kept; a call checks that every edge of the tree still holds the module it held (a replaced
    module, e.g. by another oneshot, walks again) and reads the tensors through their holders (a call costs
    ~0.1 ms of the time to first token)."""
    tree = model.__dict__.get("_llmq_module_tree")
    if not tree or not all(parent._modules.get(name) is child for parent, name, child in tree["edges"]):
        tree = _module_tree(model)
        model.__dict__["_llmq_module_tree"] = tree
    key = []
    for holder, name in tree["slots"]:
        tensor = holder.get(name)
        if tensor is None:
            key.append(None)
        else:
            key.append((tensor.data_ptr(), tensor._version, tensor.dtype))
    return tuple(key)


def kept_kernel_runtime(model, max_len: int, kv_bits: int = 8):
    """kernel_runtime, kept on the model between generate calls together with its captured step (which
    reads token and position from the device, so it serves any prompt that fits max_len): a serving
    loop does not rebuild and re-capture per request. Up to _KEPT_RUNTIMES cache lengths are kept; a
    change of any parameter or buffer of the model drops them all."""
    weights = _weights_key(model)
    kept = model.__dict__.get("_llmq_kept_runtimes")
    if not kept or kept["weights"] != weights:
        kept = _Kept(weights=weights, runtimes={})
        model.__dict__["_llmq_kept_runtimes"] = kept
    runtimes = kept["runtimes"]
    key = (max_len, kv_bits)
    runtime = runtimes.pop(key, None)
    if runtime is None:
        runtime = kernel_runtime(model, max_len, kv_bits)
        while len(runtimes) >= _KEPT_RUNTIMES:
            runtimes.pop(next(iter(runtimes)))  # the least recently used
    runtimes[key] = runtime  # most recently used last
    return runtime


def drop_kept(model) -> None:
    """Forget everything graphed_generate keeps on `model` (up to four runtimes per side, each with its KV cache
    and the memory pool of its captured graph; they reference the model and the model them, so without this
    they live until the cycle collector finds the model unreachable)."""
    for name in ("_llmq_kept_runtimes", "_llmq_kept_decoders", "_llmq_module_tree"):
        model.__dict__.pop(name, None)


def kept_graphed_decoder(model, prompt_tokens: int, new_tokens: int):
    """A GraphedDecoder (HF module walk over a StaticCache) kept on the model between generate calls with
    its captured step, exactly as kept_kernel_runtime keeps the kernel runtime: the captured step reads the
    token, the position and the cache length from the device, so after the first call a generate is cache
    reset + eager prompt pass + replays, on this side as on the kernel side. Keyed by the run's lengths;
    dropped when any parameter or buffer of the model changes."""
    weights = _weights_key(model)
    kept = model.__dict__.get("_llmq_kept_decoders")
    if not kept or kept["weights"] != weights:
        kept = _Kept(weights=weights, decoders={})
        model.__dict__["_llmq_kept_decoders"] = kept
    decoders = kept["decoders"]
    key = (prompt_tokens, new_tokens)
    decoder = decoders.pop(key, None)
    if decoder is None:
        decoder = GraphedDecoder(model, prompt_tokens, new_tokens)
        while len(decoders) >= _KEPT_RUNTIMES:
            decoders.pop(next(iter(decoders)))
    decoders[key] = decoder
    return decoder


class KernelDecoder:
    """Same interface over LlamaKernelRuntime and the integer KV cache."""

    def __init__(self, model, prompt_tokens: int, new_tokens: int, kv_bits: int = 8):
        self.max_len = prompt_tokens + new_tokens + 1
        self.runtime = kernel_runtime(model, self.max_len, kv_bits)
        self.graph = None

    @property
    def logits(self):
        return self.runtime.logits

    def prefill(self, input_ids):
        return self.runtime.prefill(input_ids).reshape(1, 1)

    def capture(self, position: int, token=None):
        self.runtime.capture(self.runtime.token if token is None else token, position)
        self.graph = self.runtime.graph

    def step(self, token=None, position: int | None = None):
        # the previous step already left its argmax and the advanced position on the device;
        # explicit arguments re-seed them (used when a caller rewinds or substitutes a token)
        if token is not None and position is not None and position != self.runtime.cache.get_seq_length():
            self.runtime._set_step_inputs(token, position)
        return self.runtime.step().reshape(1, 1)


@torch.no_grad()
def graphed_generate(model, input_ids, max_new_tokens: int, kv_bits: int | None = None):
    """Greedy generation with the decode step replayed; None if it cannot be graphed. Returns
    the full sequence like model.generate(..., do_sample=False). With kv_bits the integer KV
    cache and the kernel runtime are used (Llama-architecture models)."""
    if not can_graph(model):
        return None
    prompt = input_ids.shape[1]
    if kv_bits is not None:
        return kept_kernel_runtime(model, prompt + max_new_tokens + 1, kv_bits).generate(input_ids, max_new_tokens,
                                                                                         use_graph=True)
    decoder = kept_graphed_decoder(model, prompt, max_new_tokens)
    decoder.cache.reset()
    nxt = decoder.prefill(input_ids)
    out = [nxt]
    if max_new_tokens > 1:
        decoder.token.copy_(nxt.reshape(1, 1))
        if decoder.graph is None:
            decoder.capture(prompt)
        for i in range(1, max_new_tokens):
            nxt = decoder.step(nxt, prompt + i - 1)
            out.append(nxt)
    return torch.cat([input_ids, *out], dim=1)
