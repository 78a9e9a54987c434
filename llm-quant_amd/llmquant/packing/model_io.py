"""A whole kernel-mode model in one packed file, and back (llmquant/packing/model_io.py).

File contents, in this order (key order is part of the format: the header is json.dumps of
dicts filled in this sequence):
  per quantized Linear   "<name>.qweight" (nibble-packed uint8 for 4 bit, int8 for 8 bit, in the
                         canonical [N, G, gs(/2)] layout), "<name>.wscale" (fp32), "<name>.bias"
  every other state_dict tensor as bfloat16
  non-persistent buffers (e.g. rotary inv_freq) in their own dtype
meta: model_id, layers{name: in/out features, canonical_shape, weights{...}, input_activations,
bias}, experts{name: num_experts, hidden_dim, intermediate_dim, gate_up_shape, down_shape,
weights, input_activations} (a Mixture-of-Experts block is written as one entry with its two
stacked tensors "<name>.qgate_up" / "<name>.qdown" packed like a Linear's and their scales
"<name>.sgate_up" / "<name>.sdown"), non_persistent_buffers, kv_cache_bits, plus caller extras.

Loading goes straight to the HBM layout: a 4-bit layer's packed bytes are handed to
KernelQuantLinear as they are (the reference unpacks them back to one code per byte,
model_io.py:174-189), so nothing wider than the file ever exists on the device.
"""

from __future__ import annotations

import torch
import torch.nn as nn

from llmquant.core.scheme import QuantizationArgs, QuantizationScheme
from llmquant.packing.format import read_header, read_packed, write_packed
from llmquant.packing.packing import pack_weight
from llmquant.quantizers.experts import KernelQuantExperts
from llmquant.quantizers.kernel import KernelQuantLinear

_ARG_FIELDS = ("num_bits", "strategy", "group_size", "head_dim", "out_group", "symmetric", "dynamic")


def _args_to_dict(args):
    return None if args is None else {field: getattr(args, field) for field in _ARG_FIELDS}


def _args_from_dict(payload):
    return None if payload is None else QuantizationArgs(**payload)


def _quantized_layers(model):
    return [(name, m) for name, m in model.named_modules() if isinstance(m, KernelQuantLinear)]


def save_packed_model(model: nn.Module, path, model_id: str, kv_cache_bits=None, extra=None):
    """Write every weight of a kernel-mode model into one file; returns the path."""
    tensors, layers = {}, {}
    for name, module in _quantized_layers(model):
        args = module.scheme.weights
        # module.qdata already is pack_weight(module.qweight, bits): same bytes, no round trip
        stored = module.qdata if module.qdata.dtype == torch.uint8 else pack_weight(module.qdata, args.num_bits)
        canonical_shape = list(stored.shape)
        if stored.dtype == torch.uint8:
            canonical_shape[-1] *= 2
        tensors[f"{name}.qweight"] = stored
        tensors[f"{name}.wscale"] = module.wscale
        layers[name] = {
            "in_features": module.in_features,
            "out_features": module.out_features,
            "canonical_shape": canonical_shape,
            "weights": _args_to_dict(args),
            "input_activations": _args_to_dict(module.scheme.input_activations),
            "bias": module.bias is not None,
        }
        if module.bias is not None:
            tensors[f"{name}.bias"] = module.bias

    experts = {}
    for name, module in model.named_modules():
        if not isinstance(module, KernelQuantExperts):
            continue
        args = module.scheme.weights

        def canonical(shape, packed):
            return [*shape[:-1], shape[-1] * 2] if packed else list(shape)

        packed = module.gate_up_data.dtype == torch.uint8
        tensors[f"{name}.qgate_up"] = module.gate_up_data  # already pack_weight(canonical, bits)
        tensors[f"{name}.sgate_up"] = module.sgate_up
        tensors[f"{name}.qdown"] = module.down_data
        tensors[f"{name}.sdown"] = module.sdown
        experts[name] = {
            "num_experts": module.num_experts,
            "hidden_dim": module.hidden_dim,
            "intermediate_dim": module.intermediate_dim,
            "gate_up_shape": canonical(module.gate_up_data.shape, packed),
            "down_shape": canonical(module.down_data.shape, packed),
            "weights": _args_to_dict(args),
            "input_activations": _args_to_dict(module.scheme.input_activations),
        }

    # whatever a quantized layer owns (stored or derived) is excluded by prefix, so a derived
    # buffer can never be written as bf16 and later overwrite its exactly computed value
    owned = tuple(f"{name}." for name in (*layers, *experts))
    # (the quantized modules' own state_dict form unpacks 4-bit codes: walk the other modules only)
    state = {}
    for prefix, module in model.named_modules():
        full = f"{prefix}." if prefix else ""
        if not full.startswith(owned):
            module._save_to_state_dict(state, full, keep_vars=False)
    for name, tensor in state.items():
        if name.startswith(owned) or name in tensors:
            continue
        tensors[name] = tensor.detach().to(torch.bfloat16)

    non_persistent = []
    for name, buffer in model.named_buffers():
        if name.startswith(owned) or name in state or name in tensors:
            continue
        tensors[name] = buffer.detach()
        non_persistent.append(name)

    meta = {"model_id": model_id, "layers": layers, "experts": experts, "non_persistent_buffers": non_persistent,
            "kv_cache_bits": kv_cache_bits, **(extra or {})}
    return write_packed(path, tensors, meta)


def _set_submodule(model, dotted, module):
    owner, _, leaf = dotted.rpartition(".")
    setattr(model.get_submodule(owner) if owner else model, leaf, module)


def _give_storage_to_meta_leftovers(model, device, dtype, provided):
    """Allocate only what is still on `meta` and will not be assigned from the file; the
    quantized modules already hold real tensors and must not be touched."""
    for prefix, module in model.named_modules():
        for name, param in list(module.named_parameters(recurse=False)):
            full = f"{prefix}.{name}" if prefix else name
            if param is not None and param.is_meta and full not in provided:
                fresh = torch.empty(param.shape, dtype=dtype, device=device)
                setattr(module, name, nn.Parameter(fresh, requires_grad=param.requires_grad))
        for name, buffer in list(module.named_buffers(recurse=False)):
            full = f"{prefix}.{name}" if prefix else name
            if buffer is not None and buffer.is_meta and full not in provided:
                persistent = name not in getattr(module, "_non_persistent_buffers_set", set())
                module.register_buffer(name, torch.empty(buffer.shape, dtype=buffer.dtype, device=device),
                                       persistent=persistent)


def load_packed_model(path, device="cuda", dtype=torch.bfloat16, config=None):
    """Rebuild the model from a packed file without ever materialising bf16 weights for the
    quantized layers. The architecture comes from `config`, or from
    AutoConfig.from_pretrained(meta["model_id"]) (a local path works offline)."""
    from transformers import AutoConfig, AutoModelForCausalLM

    tensors, meta = read_packed(path)
    if config is None:
        config = AutoConfig.from_pretrained(meta["model_id"])
    with torch.device("meta"):
        model = AutoModelForCausalLM.from_config(config)

    for name, spec in meta["layers"].items():
        args = _args_from_dict(spec["weights"])
        scheme = QuantizationScheme(weights=args, input_activations=_args_from_dict(spec["input_activations"]))
        stored = tensors[f"{name}.qweight"]
        shape = list(spec["canonical_shape"])
        if stored.dtype == torch.uint8:
            shape[-1] //= 2  # stays packed: this is the HBM layout
        else:
            stored = stored.to(torch.int8)
        bias = tensors.get(f"{name}.bias")
        module = KernelQuantLinear(
            stored.reshape(shape).to(device), tensors[f"{name}.wscale"].to(device),
            nn.Parameter(bias.to(device=device, dtype=dtype)) if bias is not None else None,
            scheme, spec["in_features"])
        _set_submodule(model, name, module)

    for name, spec in (meta.get("experts") or {}).items():
        args = _args_from_dict(spec["weights"])
        scheme = QuantizationScheme(weights=args, input_activations=_args_from_dict(spec["input_activations"]))

        def stack(key, shape):
            stored = tensors[f"{name}.{key}"]
            shape = list(shape)
            if stored.dtype == torch.uint8:
                shape[-1] //= 2  # stays packed
            else:
                stored = stored.to(torch.int8)
            return stored.reshape(shape).to(device)

        # the activation function is architecture, not weights: taken from the block being replaced
        module = KernelQuantExperts(stack("qgate_up", spec["gate_up_shape"]), tensors[f"{name}.sgate_up"].to(device),
                                    stack("qdown", spec["down_shape"]), tensors[f"{name}.sdown"].to(device), scheme,
                                    spec["hidden_dim"], spec["intermediate_dim"], model.get_submodule(name).act_fn)
        _set_submodule(model, name, module)

    _give_storage_to_meta_leftovers(model, device, dtype, provided=set(tensors))
    non_persistent = set(meta.get("non_persistent_buffers", []))
    owned = tuple(f"{name}." for name in (*meta["layers"], *(meta.get("experts") or {})))
    rest = {name: t.to(device=device, dtype=dtype) for name, t in tensors.items()
            if name not in non_persistent and not name.startswith(owned)}
    _, unexpected = model.load_state_dict(rest, strict=False, assign=True)
    unexpected = [n for n in unexpected if not n.startswith(owned)]
    if unexpected:
        raise ValueError(f"packed file has tensors the model does not want: {unexpected[:5]}")
    for name in non_persistent:
        owner, _, leaf = name.rpartition(".")
        (model.get_submodule(owner) if owner else model).register_buffer(leaf, tensors[name].to(device),
                                                                         persistent=False)
    return model.eval()


def packed_dtypes(path) -> dict:
    """The dtype each axis actually has in a packed file, read from the header."""
    meta = read_header(path)["meta"]
    seen = {"attn_weight": set(), "mlp_weight": set(), "head_weight": set()}
    for name, spec in (meta.get("layers") or {}).items():
        axis = ("attn_weight" if ".self_attn." in name else "mlp_weight" if ".mlp." in name
                else "head_weight" if "lm_head" in name else None)
        bits = (spec.get("weights") or {}).get("num_bits")
        if axis and bits:
            seen[axis].add(bits)

    def label(bits):
        return "bf16" if not bits else "mixed" if len(bits) > 1 else f"int{next(iter(bits))}"

    kv_bits = meta.get("kv_cache_bits")
    return {**{axis: label(bits) for axis, bits in seen.items()},
            "kv_cache": f"int{kv_bits}" if kv_bits else "bf16",
            "activation": "bf16"}


def describe_packed(path) -> dict:
    header = read_header(path)
    entries = header["tensors"]
    return {"model_id": header["meta"]["model_id"], "quantized_layers": len(header["meta"]["layers"]),
            "tensors": len(entries), "bytes": sum(e["nbytes"] for e in entries.values())}
