"""CPU oracle for llm-quant's `mode="kernel"` path -- TEST INFRASTRUCTURE, not product code.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module;
the shipped package never does, and never falls back to it.

It restates, in plain numpy with every rounding point made explicit, what the reference
computes on this path. Each function names the reference source it follows. Arrays carry
values as float32 (or integer) numpy arrays; a `dtype` tag ("f32" | "f16" | "bf16") says
which storage type a result must be rounded to, because numpy has no bfloat16.

What pins each function (the tests that do so live in tests/test_oracle_*.py):
  round_to / bf16      known bit patterns, ties, torch CPU casts as an independent check
  compute_scale        true-division constant, shape table, eps floor    (reference tests/test_quantization.py:13-84)
  quantize             half-to-even list, abs-max -> +-qmax, range       (same file)
  fake_quantize        padding-free, channel == group=K, idempotence, torch CPU restatement
  group_view & co      shape table and round trips                        (reference tests/test_grouping.py)
  quantize_weight      range/shape facts + per-group python loops        (reference tests/test_real_quant.py:24-30)
  real_linear          exact int64 group sums, float64 closed form, tracks fake   (reference tests/test_real_quant.py:33-99)
  pack_int4            0xD5 example, exhaustive round trip                 (reference tests/test_packing.py:31-46)
  write_packed         magic / version / alignment / round trip            (reference tests/test_packing.py:65-101)
  kv_quant             == fake_quantize at group 64; old tokens untouched  (reference tests/test_kv_cache.py)
  route_plan           brute force over every row: coverage once, no run over two experts, run length
                       (reference tests/test_moe.py:310-333)
  moe_experts_real     per expert == real_linear; tracks transformers' MixtralExperts in bf16
                       (reference tests/test_moe.py:77-117, 336-345)
  llama_rmsnorm, llama_gated_act, llama_residual_add
                       the elementwise steps of transformers' LlamaDecoderLayer around the Linears
                       (third-party arithmetic the reference delegates to); pinned against the library's own
                       LlamaRMSNorm / LlamaMLP modules and torch's bf16/fp16 adds on the CPU, and by closed
                       forms (a constant row normalises to +-weight, silu(0) = 0)
  gqa_decode_attention the reference delegates attention to HF transformers and holds no test of its
                       arithmetic; pinned against the routines it delegates to (transformers'
                       eager_attention_forward and torch's scaled_dot_product_attention, grouped-query,
                       on the CPU) and by closed forms (uniform scores -> mean of V, one dominant key).
"""

from __future__ import annotations

import json
import struct

import numpy as np

SCALE_EPS = np.float32(1e-8)  # llmquant/core/observers.py:5
GROUP_SIZE = 128  # llmquant/core/scheme.py:3
INT4_BIAS = 8  # llmquant/packing/packing.py:16

# ---------------------------------------------------------------------------------------------
# storage types
# ---------------------------------------------------------------------------------------------


def bf16_bits(x) -> np.ndarray:
    """float32 -> the 16 bits of the nearest bfloat16, ties to even (NaN -> 0x7fc0)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    rounded = (u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    return np.where(nan, np.uint32(0x7FC0), rounded).astype(np.uint16)


def bf16_from_bits(bits) -> np.ndarray:
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def round_to(x, dtype: str) -> np.ndarray:
    """Round float32 values to what `dtype` can store, returned as float32."""
    x = np.asarray(x, dtype=np.float32)
    if dtype == "f32":
        return x
    if dtype == "f16":
        with np.errstate(over="ignore"):
            return x.astype(np.float16).astype(np.float32)
    if dtype == "bf16":
        return bf16_from_bits(bf16_bits(x)).reshape(x.shape)
    raise ValueError(f"unknown dtype tag {dtype!r}")


# ---------------------------------------------------------------------------------------------
# grouping geometry -- llmquant/core/observers.py:8-71
# ---------------------------------------------------------------------------------------------


def pad_to_group(x: np.ndarray, group_size: int) -> np.ndarray:
    """Zero-pad the last axis to a multiple of group_size (observers.py:8-20)."""
    rem = x.shape[-1] % group_size
    if rem == 0:
        return x
    widths = [(0, 0)] * (x.ndim - 1) + [(0, group_size - rem)]
    return np.pad(x, widths)


def group_view(x: np.ndarray, group_size: int, head_dim: int | None = None) -> np.ndarray:
    """[..., K] -> [..., groups, group_size]; with head_dim each head is padded on its own
    (observers.py:23-43)."""
    if head_dim is None:
        p = pad_to_group(x, group_size)
        return p.reshape(*p.shape[:-1], p.shape[-1] // group_size, group_size)
    lead, k = x.shape[:-1], x.shape[-1]
    if k % head_dim:
        raise ValueError(f"last dim {k} is not a multiple of head_dim {head_dim}")
    heads = pad_to_group(x.reshape(*lead, k // head_dim, head_dim), group_size)
    return heads.reshape(*lead, -1, group_size)


def ungroup(y: np.ndarray, shape, group_size: int, head_dim: int | None = None) -> np.ndarray:
    """Inverse of group_view, dropping the padding (observers.py:46-53)."""
    lead, k = tuple(shape[:-1]), shape[-1]
    if head_dim is None:
        return y.reshape(*lead, -1)[..., :k]
    padded_head = -(-head_dim // group_size) * group_size
    return y.reshape(*lead, k // head_dim, padded_head)[..., :head_dim].reshape(*lead, k)


def out_block_view(x: np.ndarray, out_group: int) -> np.ndarray:
    """[out, ...] -> [ceil(out/out_group), out_group, ...], zero-padded (observers.py:56-66)."""
    rem = x.shape[0] % out_group
    if rem:
        x = np.pad(x, [(0, out_group - rem)] + [(0, 0)] * (x.ndim - 1))
    return x.reshape(-1, out_group, *x.shape[1:])


def out_unblock(y: np.ndarray, out: int) -> np.ndarray:
    return y.reshape(-1, *y.shape[2:])[:out]


# ---------------------------------------------------------------------------------------------
# the quantizer -- llmquant/core/observers.py:74-98, llmquant/core/quant_ops.py:13-37
# ---------------------------------------------------------------------------------------------


def qrange(num_bits: int):
    qmax = 2 ** (num_bits - 1) - 1
    return -qmax - 1, qmax


def compute_scale(x, num_bits, strategy="group", group_size=None, head_dim=None, out_group=None):
    """Symmetric abs-max scale, fp32, keepdim (observers.py:74-98).

    amax / qmax is a true IEEE fp32 division (numpy's float32 `/` is one), then floored at
    SCALE_EPS.
    """
    _, qmax = qrange(num_bits)
    xf = np.asarray(x, dtype=np.float32)
    if strategy == "group":
        view = group_view(xf, group_size, head_dim)
        if out_group:
            amax = np.abs(out_block_view(view, out_group)).max(axis=(1, -1), keepdims=True)
        else:
            amax = np.abs(view).max(axis=-1, keepdims=True)
    elif strategy in ("channel", "token"):
        amax = np.abs(xf).max(axis=-1, keepdims=True)
    else:
        raise ValueError(f"unsupported strategy {strategy!r}")
    scale = amax.astype(np.float32) / np.float32(qmax)
    return np.maximum(scale, SCALE_EPS).astype(np.float32)


def quantize(x, scale, num_bits) -> np.ndarray:
    """Integer-valued float32: clamp(rint(x / scale)) with ties to even (quant_ops.py:13-19)."""
    qmin, qmax = qrange(num_bits)
    with np.errstate(over="ignore", invalid="ignore"):
        q = np.rint(np.asarray(x, dtype=np.float32) / np.asarray(scale, dtype=np.float32))
    return np.clip(q, np.float32(qmin), np.float32(qmax)).astype(np.float32)


def dequantize(q, scale) -> np.ndarray:
    return (np.asarray(q, dtype=np.float32) * np.asarray(scale, dtype=np.float32)).astype(np.float32)


def fake_quantize(x, num_bits, dtype="f32", strategy="group", group_size=None, head_dim=None,
                  out_group=None) -> np.ndarray:
    """Quantize-dequantize, rounded back to `dtype` (quant_ops.py:26-37)."""
    x = np.asarray(x, dtype=np.float32)
    scale = compute_scale(x, num_bits, strategy, group_size, head_dim, out_group)
    if strategy != "group":
        return round_to(dequantize(quantize(x, scale, num_bits), scale), dtype)
    view = group_view(x, group_size, head_dim)
    if out_group:
        blocked = out_block_view(view, out_group)
        out = out_unblock(dequantize(quantize(blocked, scale, num_bits), scale), x.shape[0])
    else:
        out = dequantize(quantize(view, scale, num_bits), scale)
    return round_to(ungroup(out, x.shape, group_size, head_dim), dtype)


def quant_group_codes(x, num_bits, group_size):
    """(codes int8 [..., K], scale fp32 [..., K/gs]) for a last axis that is a whole number of
    groups: the op the fused kernel implements."""
    x = np.asarray(x, dtype=np.float32)
    if x.shape[-1] % group_size:
        raise ValueError("last dim must be a multiple of group_size")
    scale = compute_scale(x, num_bits, "group", group_size)
    q = quantize(group_view(x, group_size), scale, num_bits)
    return q.reshape(x.shape).astype(np.int8), scale[..., 0]


# ---------------------------------------------------------------------------------------------
# weights -- llmquant/quantizers/real.py:29-47, llmquant/quantizers/kernel.py:56-66
# ---------------------------------------------------------------------------------------------


def quantize_weight(weight, num_bits, group_size=GROUP_SIZE, head_dim=None, out_group=None):
    """(codes int8 [out, in], scale fp32 keepdim) (real.py:29-47)."""
    w = np.asarray(weight, dtype=np.float32)
    scale = compute_scale(w, num_bits, "group", group_size, head_dim, out_group)
    grouped = group_view(w, group_size, head_dim)
    if out_group:
        q = out_unblock(quantize(out_block_view(grouped, out_group), scale, num_bits), w.shape[0])
    else:
        q = quantize(grouped, scale, num_bits)
    q = ungroup(q, w.shape, group_size, head_dim)
    return q.astype(np.int8), scale


def canonical_weight(weight, num_bits, group_size=GROUP_SIZE, head_dim=None, out_group=None):
    """What KernelQuantLinear.from_linear stores (kernel.py:56-66): codes [N, G, gs] int8
    with padding and head split baked in, scales [scale_rows, G] fp32."""
    q, scale = quantize_weight(weight, num_bits, group_size, head_dim, out_group)
    canonical = np.ascontiguousarray(group_view(q, group_size, head_dim))
    flat_scale = np.ascontiguousarray(scale.reshape(-1, canonical.shape[1]).astype(np.float32))
    return canonical, flat_scale


def pad_activation(flat, group_size=GROUP_SIZE, head_dim=None):
    """Activation padded the way the weight was (kernel.py:17-25)."""
    if head_dim:
        lead, k = flat.shape[:-1], flat.shape[-1]
        heads = pad_to_group(flat.reshape(*lead, k // head_dim, head_dim), group_size)
        return heads.reshape(*lead, -1)
    return pad_to_group(flat, group_size)


def _row_scale(wscale2d, n_rows, out_group):
    """[scale_rows, G] -> [N, G] by repeating each scale row over its output tile."""
    if out_group:
        return np.repeat(wscale2d, out_group, axis=0)[:n_rows]
    return wscale2d


def real_linear(x, canonical, wscale2d, dtype="f32", out_group=None, act_bits=None, bias=None):
    """RealQuantLinear.forward on canonical operands (real.py:76-103).

    x: [M, G*gs] float32 values already padded like the weight. For every group, in order:
    partial = x_g @ q_g^T  -> * s_w  [-> * s_x] -> out += partial, each step rounded to fp32.
    With act_bits the activation is quantized per token x group first and the integer
    product is exact; without it the in-group sum is taken in float64 and rounded once,
    which no fp32 summation order can beat (the reference leaves that order to the BLAS).
    """
    x = np.asarray(x, dtype=np.float32)
    n, groups, gs = canonical.shape
    m = x.shape[0]
    xg = x.reshape(m, groups, gs)
    sw = _row_scale(np.asarray(wscale2d, dtype=np.float32), n, out_group)  # [N, G]
    if act_bits is None:
        sx = None
        a = xg.astype(np.float64)
    else:
        sx = compute_scale(x, act_bits, "group", gs)  # [M, G, 1]
        a = quantize(xg, sx, act_bits).astype(np.int64)
    out = np.zeros((m, n), dtype=np.float32)
    for g in range(groups):
        if act_bits is None:
            partial = (a[:, g] @ canonical[:, g].astype(np.float64).T).astype(np.float32)
        else:
            partial = (a[:, g] @ canonical[:, g].astype(np.int64).T).astype(np.float32)
        partial = partial * sw[None, :, g]
        if sx is not None:
            partial = partial * sx[:, g]
        out = out + partial.astype(np.float32)
    if bias is not None:
        out = out + np.asarray(bias, dtype=np.float32)
    return round_to(out, dtype)


def dequantized_weight(canonical, wscale2d, dtype="bf16", out_group=None):
    """KernelQuantLinear._dequantized_weight (kernel.py:68-79): (q * s) rounded to dtype,
    [N, G*gs]."""
    n = canonical.shape[0]
    sw = _row_scale(np.asarray(wscale2d, dtype=np.float32), n, out_group)
    w = canonical.astype(np.float32) * sw[:, :, None]
    return round_to(w, dtype).reshape(n, -1)


def gemv_float64(x, canonical, wscale2d, out_group=None):
    """The closed form sum_g s_g * sum_k x_k q_k in float64: the tolerance anchor."""
    n = canonical.shape[0]
    sw = _row_scale(np.asarray(wscale2d, dtype=np.float64), n, out_group)
    w = canonical.astype(np.float64) * sw[:, :, None]
    return np.asarray(x, dtype=np.float64) @ w.reshape(n, -1).T


# ---------------------------------------------------------------------------------------------
# Mixture-of-Experts -- llmquant/quantizers/real.py:117-190, llmquant/quantizers/kernel.py:176-214
# ---------------------------------------------------------------------------------------------


def route_plan(top_k_index, num_experts: int, limit: int):
    """KernelQuantExperts._plan (kernel.py:176-214) with python loops: rows sorted by expert
    (stable), every expert given ceil(rows / limit) blocks of at most `limit` rows."""
    flat = np.asarray(top_k_index).reshape(-1)
    order = np.argsort(flat, kind="stable")
    per_expert = max(1, -(-flat.size // limit))
    expert, row0, length = [], [], []
    start = 0
    for e in range(num_experts):
        count = int((flat == e).sum())
        for b in range(per_expert):
            expert.append(e)
            row0.append(start + b * limit)
            length.append(min(max(count - b * limit, 0), limit))
        start += count
    return order, (np.array(expert), np.array(row0), np.array(length))


def silu(x, dtype="bf16"):
    xf = np.asarray(x, dtype=np.float32)
    return round_to(xf / (1.0 + np.exp(-xf.astype(np.float64))).astype(np.float32), dtype)


def moe_experts_real(hidden, top_k_index, top_k_weights, qgate_up, sgate_up, qdown, sdown, dtype="bf16"):
    """RealQuantExperts.forward (real.py:160-190): experts in ascending order; for each, the
    tokens routed to it go through gate_up -> silu(gate) * up -> down as dequantize-then-fp32
    matmuls with the result rounded to `dtype` after each (here the products are summed in
    float64 and rounded once), are scaled by the routing weight and added into the output.
    hidden [T, H] float32 holding `dtype` values; codes [E, N, G, gs]; scales [E, rows, G]."""
    hidden = np.asarray(hidden, dtype=np.float32)
    index = np.asarray(top_k_index)
    weights = np.asarray(top_k_weights, dtype=np.float32)
    final = np.zeros_like(hidden)
    h_dim = hidden.shape[1]

    def project(x, codes, scales):
        n = codes.shape[0]
        w = codes.astype(np.float64) * _row_scale(scales.astype(np.float64), n, codes.shape[0] // scales.shape[0]
                                                  if scales.shape[0] != n else None)[:, :, None]
        w = w.reshape(n, -1)[:, : x.shape[1]]
        return round_to((x.astype(np.float64) @ w.T).astype(np.float32), dtype)

    for e in range(qgate_up.shape[0]):
        token, slot = np.nonzero(index == e)
        if token.size == 0:
            continue
        fused = project(hidden[token], qgate_up[e], sgate_up[e])
        half = fused.shape[1] // 2
        act = round_to(silu(fused[:, :half], dtype) * fused[:, half:], dtype)
        out = project(act, qdown[e], sdown[e])
        out = round_to(out * weights[token, slot, None], dtype)
        final[token] = round_to(final[token] + out, dtype)
    assert final.shape[1] == h_dim
    return final


# ---------------------------------------------------------------------------------------------
# The elementwise steps of a decoder layer around the quantized Linears. The reference runs them through HF
# transformers (LlamaDecoderLayer; installed transformers/models/llama/modeling_llama.py: LlamaRMSNorm.forward,
# LlamaMLP.forward, the residual adds of LlamaDecoderLayer.forward). Rounding points are the library's.
# ---------------------------------------------------------------------------------------------


def llama_rmsnorm(x, weight, eps, dtype="bf16"):
    """LlamaRMSNorm.forward: x to fp32, variance = mean(x^2) over the last axis, x * rsqrt(variance + eps),
    rounded to `dtype`, then weight * that, rounded to `dtype` again. The mean is taken in float64 and
    rounded to fp32 once (torch leaves its order to the reduction kernel)."""
    xf = np.asarray(x, dtype=np.float32)
    variance = (xf.astype(np.float64) ** 2).mean(axis=-1, keepdims=True).astype(np.float32)
    inv = (1.0 / np.sqrt((variance + np.float32(eps)).astype(np.float64))).astype(np.float32)
    normed = round_to(xf * inv, dtype)
    return round_to(np.asarray(weight, dtype=np.float32) * normed, dtype)


def llama_gated_act(gate, up, dtype="bf16"):
    """LlamaMLP.forward's act_fn(gate_proj(x)) * up_proj(x) on `dtype` tensors: silu rounded to `dtype`, the
    product rounded to `dtype`."""
    return round_to(silu(gate, dtype) * np.asarray(up, dtype=np.float32), dtype)


def llama_residual_add(residual, branch, dtype="bf16"):
    """residual + branch on `dtype` tensors (LlamaDecoderLayer.forward): one rounding of the exact sum."""
    return round_to(np.asarray(residual, dtype=np.float32) + np.asarray(branch, dtype=np.float32), dtype)


# ---------------------------------------------------------------------------------------------
# packing -- llmquant/packing/packing.py:16-57, llmquant/packing/format.py:29-118
# ---------------------------------------------------------------------------------------------


def pack_int4(values) -> np.ndarray:
    """int8 in [-8, 7] -> uint8, +8 bias, even index in the low nibble (packing.py:20-33)."""
    v = np.asarray(values)
    if v.shape[-1] % 2:
        raise ValueError(f"last dim {v.shape[-1]} must be even to pack into nibbles")
    if v.size and (v.min() < -8 or v.max() > 7):
        raise ValueError(f"values must be in [-8, 7], got [{int(v.min())}, {int(v.max())}]")
    biased = (v.astype(np.int16) + INT4_BIAS).astype(np.uint8)
    return np.ascontiguousarray(biased[..., 0::2] | (biased[..., 1::2] << 4))


def unpack_int4(packed) -> np.ndarray:
    p = np.asarray(packed, dtype=np.uint8)
    low = (p & 0x0F).astype(np.int16) - INT4_BIAS
    high = ((p >> 4) & 0x0F).astype(np.int16) - INT4_BIAS
    return np.stack((low, high), axis=-1).reshape(*p.shape[:-1], -1).astype(np.int8)


MAGIC = b"LLMQUANT"
VERSION = 1
ALIGNMENT = 64


def packed_file_bytes(tensors: dict, meta: dict) -> bytes:
    """The bytes write_packed produces (format.py:65-93). `tensors` maps name ->
    (dtype_name, numpy array); bfloat16 tensors are passed as their uint16 bit patterns."""
    entries, blobs, offset = {}, [], 0
    for name, (dtype_name, array) in tensors.items():
        payload = np.ascontiguousarray(array).tobytes()
        pad = -offset % ALIGNMENT
        if pad:
            blobs.append(b"\0" * pad)
            offset += pad
        entries[name] = {"dtype": dtype_name, "shape": list(array.shape), "offset": offset,
                         "nbytes": len(payload)}
        blobs.append(payload)
        offset += len(payload)
    header = json.dumps({"version": VERSION, "meta": meta, "tensors": entries}).encode("utf-8")
    return MAGIC + struct.pack("<Q", len(header)) + header + b"".join(blobs)


# ---------------------------------------------------------------------------------------------
# KV cache -- llmquant/quantizers/fake.py:39-55
# ---------------------------------------------------------------------------------------------


def kv_quant(states, num_bits):
    """Per token, per head: (codes int8 [..., D], scale fp32 [...]) for head_dim D <= 128.

    FakeQuantCache groups the last axis at 128 with zero padding, which for D <= 128 is one
    group per (token, head) whose scale only sees the D real values.
    """
    s = np.asarray(states, dtype=np.float32)
    if s.shape[-1] > GROUP_SIZE:
        raise ValueError("head_dim above the group size needs more than one scale per token")
    scale = compute_scale(s, num_bits, "group", GROUP_SIZE)  # [..., 1, 1]
    q = quantize(group_view(s, GROUP_SIZE), scale, num_bits)
    return ungroup(q, s.shape, GROUP_SIZE).astype(np.int8), scale[..., 0, 0]


def kv_dequant(codes, scale, dtype="bf16"):
    """What FakeQuantCache stores: (q * scale) rounded to the cache dtype."""
    return round_to(codes.astype(np.float32) * np.asarray(scale, dtype=np.float32)[..., None], dtype)


def gqa_decode_attention(q, k, v, sm_scale, dtype="bf16"):
    """One query token against the whole cache, grouped-query. q: [Hq, D]; k, v: [Hkv, T, D]
    (already dequantized values). softmax(q k^T * sm_scale) v in float64, rounded to dtype."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    hq, hkv = q.shape[0], k.shape[0]
    rep = hq // hkv
    out = np.zeros_like(q)
    for h in range(hq):
        kk, vv = k[h // rep], v[h // rep]
        s = (kk @ q[h]) * sm_scale
        p = np.exp(s - s.max())
        out[h] = (p / p.sum()) @ vv
    return round_to(out.astype(np.float32), dtype)


def gqa_prompt_attention(q, k, v, sm_scale) -> np.ndarray:
    """A whole prompt, causal and grouped-query: query i sees keys 0..i. q: [T, Hq, D]; k, v: [Hkv, T, D]
    (the values FakeQuantCache.update hands back, fake.py:39-55, which is what the reference's prompt pass
    gives transformers' attention). softmax(q k^T * sm_scale + causal mask) v in float64 -> [T, Hq * D]
    float64 (unrounded: the tolerance anchor of the GPU kernel)."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    tokens, hq, d = q.shape
    rep = hq // k.shape[0]
    out = np.zeros((tokens, hq, d))
    hidden = np.triu(np.ones((tokens, tokens), dtype=bool), 1)   # key j > query i
    for h in range(hq):
        s = (q[:, h] @ k[h // rep].T) * sm_scale
        s[hidden] = -np.inf
        p = np.exp(s - s.max(axis=1, keepdims=True))
        out[:, h] = (p / p.sum(axis=1, keepdims=True)) @ v[h // rep]
    return out.reshape(tokens, hq * d)
