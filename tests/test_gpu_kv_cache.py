"""Quantized KV cache kernels against the CPU oracle: append (codes and scales bit-exact, as
FakeQuantCache's arithmetic gives them), dequantize-on-read, and the fused single-token GQA
attention (rel-L2 <= 1e-2 for bf16 outputs, <= 1e-3 for fp32, against float64 softmax attention
over the (dtype)(code*scale) values; that attention arithmetic is not pinned by the reference,
which delegates it to HF transformers)."""

import pathlib

import numpy as np
import pytest
import torch

import llmq_oracle as oracle
from conftest import rel_l2, tag_of, to_np

pytestmark = pytest.mark.gpu
GOLD = pathlib.Path(__file__).resolve().parent / "golden" / "kv_case.npz"


@pytest.fixture(scope="module")
def ext():
    from llmquant.hip import load_extension

    return load_extension()


def new_cache(kv_heads, t_max, d, bits, dev="cuda"):
    width = d if bits == 8 else d // 2
    dt = torch.int8 if bits == 8 else torch.uint8
    return dict(k_codes=torch.zeros(kv_heads, t_max, width, dtype=dt, device=dev),
                v_codes=torch.zeros(kv_heads, t_max, width, dtype=dt, device=dev),
                k_scale=torch.zeros(kv_heads, t_max, device=dev), v_scale=torch.zeros(kv_heads, t_max, device=dev))


def append(ext, cache, k, v, pos, dq=False):
    position = torch.tensor([pos], dtype=torch.int32, device="cuda")
    return ext.kv_append(k, v, cache["k_codes"], cache["v_codes"], cache["k_scale"], cache["v_scale"], position, dq)


def codes_np(t, bits):
    a = t.cpu().numpy()
    return oracle.unpack_int4(a) if bits == 4 else a


@pytest.mark.parametrize("bits", [8, 4])
def test_golden_case(ext, bits):
    g = np.load(GOLD)
    k = torch.from_numpy(g["k"].copy()).view(torch.bfloat16).cuda()
    v = torch.from_numpy(g["v"].copy()).view(torch.bfloat16).cuda()
    q = torch.from_numpy(g["q"].copy()).view(torch.bfloat16).cuda()
    kv_heads, t, d = k.shape
    cache = new_cache(kv_heads, 64, d, bits)
    append(ext, cache, k, v, 0)
    assert np.array_equal(codes_np(cache["k_codes"], bits)[:, :t], g[f"k_codes{bits}"])
    assert np.array_equal(codes_np(cache["v_codes"], bits)[:, :t], g[f"v_codes{bits}"])
    assert np.array_equal(to_np(cache["k_scale"])[:, :t], g[f"k_scale{bits}"])
    assert np.array_equal(to_np(cache["v_scale"])[:, :t], g[f"v_scale{bits}"])
    ws = torch.zeros(ext.kv_decode_workspace_floats(q.shape[0], d, 64), device="cuda")
    length = torch.tensor([t], dtype=torch.int32, device="cuda")
    out = ext.kv_decode_attention(q, cache["k_codes"], cache["v_codes"], cache["k_scale"], cache["v_scale"], ws,
                                  length, d ** -0.5)
    assert rel_l2(to_np(out), g[f"attn{bits}"]) <= 1e-2


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("d", [64, 128])
def test_append_matches_the_oracle_and_fake_quant(ext, bits, dtype, d):
    """Prefill-shaped append: [kv_heads, T, D] taken as a strided view of [T, kv_heads, D]
    (how HF lays out projected keys), codes + scales + returned dequantized values."""
    torch.manual_seed(0)
    kv_heads, t = 8, 45
    k = (torch.randn(t, kv_heads, d) * 2).to(dtype).cuda().transpose(0, 1)
    v = torch.randn(t, kv_heads, d).to(dtype).cuda().transpose(0, 1)
    assert not k.is_contiguous()
    cache = new_cache(kv_heads, 64, d, bits)
    dq_k, dq_v = append(ext, cache, k, v, 3, dq=True)
    for name, src, dq in (("k", k, dq_k), ("v", v, dq_v)):
        want_codes, want_scale = oracle.kv_quant(to_np(src), bits)
        assert np.array_equal(codes_np(cache[f"{name}_codes"], bits)[:, 3:3 + t], want_codes)
        assert np.array_equal(to_np(cache[f"{name}_scale"])[:, 3:3 + t], want_scale)
        want_dq = oracle.fake_quantize(to_np(src), bits, tag_of(dtype), "group", 128)  # FakeQuantCache's rule
        assert dq.dtype == dtype and np.array_equal(to_np(dq).view(np.uint32), want_dq.view(np.uint32))
        assert np.all(to_np(cache[f"{name}_scale"])[:, :3] == 0) and np.all(to_np(cache[f"{name}_scale"])[:, 3 + t:] == 0)
    # dequantize-on-read of the stored range gives the same values back
    got = ext.kv_dequant(cache["k_codes"], cache["k_scale"], 3 + t, dtype)
    assert np.array_equal(to_np(got)[:, 3:], to_np(dq_k))


def test_old_tokens_are_not_requantized(ext):
    torch.manual_seed(0)
    cache = new_cache(2, 16, 64, 4)
    first = torch.randn(2, 3, 64, device="cuda", dtype=torch.bfloat16)
    append(ext, cache, first, first.clone(), 0)
    kept = {k: v.clone() for k, v in cache.items()}
    second = torch.randn(2, 2, 64, device="cuda", dtype=torch.bfloat16) * 10
    append(ext, cache, second, second.clone(), 3)
    for name in cache:
        assert torch.equal(cache[name][:, :3], kept[name][:, :3])
        assert not torch.equal(cache[name][:, 3:5], kept[name][:, 3:5])
    # positions past the end of the cache are dropped, not written out of bounds
    append(ext, cache, second, second.clone(), 15)
    assert torch.equal(cache["k_codes"][:, :3], kept["k_codes"][:, :3])


def attention_case(ext, bits, dtype, q_heads, kv_heads, d, t_max, length, seed=0):
    torch.manual_seed(seed)
    channel = torch.exp(0.5 * torch.randn(d))
    k = (torch.randn(kv_heads, length, d) * channel).to(dtype).cuda()
    v = (torch.randn(kv_heads, length, d) * channel).to(dtype).cuda()
    q = torch.randn(q_heads, d).to(dtype).cuda()
    cache = new_cache(kv_heads, t_max, d, bits)
    append(ext, cache, k, v, 0)
    ws = torch.zeros(ext.kv_decode_workspace_floats(q_heads, d, t_max), device="cuda")
    len_dev = torch.tensor([length], dtype=torch.int32, device="cuda")
    out = ext.kv_decode_attention(q, cache["k_codes"], cache["v_codes"], cache["k_scale"], cache["v_scale"], ws,
                                  len_dev, d ** -0.5)
    tag = tag_of(dtype)
    kq, ks = oracle.kv_quant(to_np(k), bits)
    vq, vs = oracle.kv_quant(to_np(v), bits)
    want = oracle.gqa_decode_attention(to_np(q), oracle.kv_dequant(kq, ks, tag), oracle.kv_dequant(vq, vs, tag),
                                       d ** -0.5, "f32")
    return out, want, (cache, ws, len_dev, q)


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("length", [1, 15, 64, 777, 2049])
def test_decode_attention_llama_1b_geometry(ext, bits, length):
    """The Llama-3.2-1B attention geometry: 32 query heads, 8 kv heads, head_dim 64, context up to 2048 + 1."""
    out, want, _ = attention_case(ext, bits, torch.bfloat16, 32, 8, 64, 2049, length)
    assert out.shape == (32, 64) and out.dtype == torch.bfloat16
    assert rel_l2(to_np(out), want) <= 1e-2


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-3), (torch.float16, 1e-2)])
@pytest.mark.parametrize("q_heads,kv_heads,d", [(8, 8, 64), (16, 8, 128), (32, 8, 128), (8, 1, 64)])
def test_decode_attention_other_geometries(ext, dtype, tol, q_heads, kv_heads, d):
    out, want, _ = attention_case(ext, 8, dtype, q_heads, kv_heads, d, 300, 211, seed=1)
    assert rel_l2(to_np(out), want) <= tol
    if dtype == torch.float32:
        assert rel_l2(to_np(out), want) <= 1e-5  # fp32 throughout: only summation order differs


def test_cost_tracks_valid_length_and_repeat_launches_agree(ext):
    """Entries beyond `length` are ignored whatever they hold, and the arrival counters are
    left clean: a second launch on the same workspace gives the same bits."""
    out, want, (cache, ws, len_dev, q) = attention_case(ext, 8, torch.bfloat16, 32, 8, 64, 1024, 100, seed=2)
    cache["k_codes"][:, 100:] = 127
    cache["k_scale"][:, 100:] = 1e6
    cache["v_codes"][:, 100:] = -128
    cache["v_scale"][:, 100:] = 1e6
    again = ext.kv_decode_attention(q, cache["k_codes"], cache["v_codes"], cache["k_scale"], cache["v_scale"], ws,
                                    len_dev, 64 ** -0.5)
    assert torch.equal(out, again)
    assert rel_l2(to_np(again), want) <= 1e-2


def test_graph_replay_follows_the_device_length(ext):
    """Append + attend captured once, replayed while position/length advance on the device;
    every replay must equal the eager result at that length."""
    torch.manual_seed(3)
    kv_heads, q_heads, d, t_max = 8, 32, 64, 256
    cache = new_cache(kv_heads, t_max, d, 8)
    ws = torch.zeros(ext.kv_decode_workspace_floats(q_heads, d, t_max), device="cuda")
    prefix = torch.randn(kv_heads, 50, d, device="cuda", dtype=torch.bfloat16)
    append(ext, cache, prefix, prefix.flip(1).contiguous(), 0)
    pos = torch.tensor([50], dtype=torch.int32, device="cuda")
    length = torch.tensor([51], dtype=torch.int32, device="cuda")
    k1 = torch.zeros(kv_heads, 1, d, device="cuda", dtype=torch.bfloat16)
    v1 = torch.zeros_like(k1)
    q = torch.zeros(q_heads, d, device="cuda", dtype=torch.bfloat16)

    def step():
        ext.kv_append(k1, v1, cache["k_codes"], cache["v_codes"], cache["k_scale"], cache["v_scale"], pos, False)
        return ext.kv_decode_attention(q, cache["k_codes"], cache["v_codes"], cache["k_scale"], cache["v_scale"], ws,
                                       length, d ** -0.5)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        k1.normal_(); v1.normal_(); q.normal_()
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = step()
    for i in range(5):
        k1.normal_(); v1.normal_(); q.normal_()
        pos.fill_(50 + i); length.fill_(51 + i)
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        eager = step()  # same inputs, same position: rewrites the same slot with the same codes
        torch.cuda.synchronize()
        assert torch.equal(got, eager), i


def test_argument_checks(ext):
    cache = new_cache(2, 16, 64, 8)
    k = torch.randn(2, 1, 64, device="cuda", dtype=torch.bfloat16)
    pos = torch.tensor([0], dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match="position must be a CUDA int32"):
        ext.kv_append(k, k, cache["k_codes"], cache["v_codes"], cache["k_scale"], cache["v_scale"], pos.long(), False)
    with pytest.raises(RuntimeError, match="cache holds"):
        ext.kv_append(k[:1], k[:1], cache["k_codes"], cache["v_codes"], cache["k_scale"], cache["v_scale"], pos, False)
    q = torch.randn(8, 64, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="workspace must be"):
        ext.kv_decode_attention(q, cache["k_codes"], cache["v_codes"], cache["k_scale"], cache["v_scale"],
                                torch.zeros(4, device="cuda"), pos, 0.125)
    ws = torch.zeros(ext.kv_decode_workspace_floats(6, 64, 16), device="cuda")
    with pytest.raises(RuntimeError, match="multiple of kv_heads|must be 1, 2, 4 or 8"):
        ext.kv_decode_attention(q[:6], cache["k_codes"], cache["v_codes"], cache["k_scale"], cache["v_scale"], ws, pos, 0.125)


# ---- the kernels the decode step runs, straight against the oracle -------------------------------------


def rope_oracle(x, cos, sin, tag="bf16"):
    """transformers' apply_rotary_pos_emb on values of the model's dtype, every product and the sum rounded to it
    (x [H, D]; cos, sin [D]): x * cos + rotate_half(x) * sin."""
    half = x.shape[-1] // 2
    rot = np.concatenate((-x[..., half:], x[..., :half]), axis=-1)
    a = oracle.round_to(x * cos, tag)
    b = oracle.round_to(rot * sin, tag)
    return oracle.round_to(a + b, tag)


DTYPE_OF_TAG = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}


def decode_step_case(ext, bits, ctx, q_heads=32, kv_heads=8, d=64, seed=0, t_max=None, tag="bf16"):
    """KV-cache quantization in decode attention, Llama-3.2-1B geometry: a cache of `ctx` tokens with
    per-channel scale variance, one new token through RoPE -> quantize-append -> attention. Returns the
    device-side cache, the q|k|v row and tables, and the oracle's attention output [Hq, D] (bf16 values)."""
    dtype = DTYPE_OF_TAG[tag]
    gen = torch.Generator().manual_seed(seed)
    channel = torch.exp(0.5 * torch.randn(d, generator=gen))
    k = (torch.randn(kv_heads, ctx, d, generator=gen) * channel).to(dtype)
    v = (torch.randn(kv_heads, ctx, d, generator=gen) * channel).to(dtype)
    qkv = torch.randn(1, (q_heads + 2 * kv_heads) * d, generator=gen).to(dtype)
    qkv[:, q_heads * d:] *= channel.repeat(2 * kv_heads).to(dtype)
    t_max = ctx + 1 if t_max is None else t_max
    inv_freq = 1.0 / (500000.0 ** (torch.arange(0, d, 2).float() / d))
    emb = torch.outer(torch.arange(t_max).float(), inv_freq)
    emb = torch.cat((emb, emb), -1)
    cos_t, sin_t = emb.cos().to(dtype), emb.sin().to(dtype)

    cache = new_cache(kv_heads, t_max, d, bits)
    if ctx:
        append(ext, cache, k.cuda(), v.cuda(), 0)

    row = to_np(qkv)[0]
    q_new = row[: q_heads * d].reshape(q_heads, d)
    k_new = row[q_heads * d: (q_heads + kv_heads) * d].reshape(kv_heads, d)
    v_new = row[(q_heads + kv_heads) * d:].reshape(kv_heads, d)
    cos, sin = to_np(cos_t)[ctx], to_np(sin_t)[ctx]
    q_rot, k_rot = rope_oracle(q_new, cos, sin, tag), rope_oracle(k_new, cos, sin, tag)
    k_all = np.concatenate((to_np(k), k_rot[:, None]), axis=1)
    v_all = np.concatenate((to_np(v), v_new[:, None]), axis=1)
    kq, ks = oracle.kv_quant(k_all, bits)
    vq, vs = oracle.kv_quant(v_all, bits)
    want = oracle.gqa_decode_attention(q_rot, oracle.kv_dequant(kq, ks, tag), oracle.kv_dequant(vq, vs, tag),
                                       d ** -0.5, tag)
    return cache, qkv.cuda(), cos_t.cuda(), sin_t.cuda(), want, (kq, ks, vq, vs)


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("ctx,splits", [(2048, 8), (2048, 16), (2048, 32), (2048, 1), (640, 8), (0, 8), (63, 8)])
def test_decode_step_attention_against_the_oracle(ext, bits, ctx, splits):
    """RoPE -> quantize-append -> split attention -> merge, the launches of the decode step, compared
    directly with the oracle (RoPE with transformers' rounding points, FakeQuantCache's codes and scales,
    float64 softmax attention over the bf16(code * scale) values): the appended codes and scales bit for
    bit, the attention output within rel-L2 1e-2, and o_proj taken as the GEMV that merges the split
    records while it stages its activation against the float64 closed form on the oracle's attention
    output. splits = 1 is the one-workgroup-per-head launch, 32 the form that shares a kv head's rows
    between its four query heads."""
    q_heads, kv_heads, d = 32, 8, 64
    cache, qkv, cos_t, sin_t, want, (kq, ks, vq, vs) = decode_step_case(ext, bits, ctx)
    position = torch.tensor([ctx], dtype=torch.int32, device="cuda")
    args = (cache["k_codes"], cache["v_codes"], cache["k_scale"], cache["v_scale"])
    if splits == 1:
        merged = ext.kv_rope_append_attend(qkv, cos_t, sin_t, *args, position, d ** -0.5, q_heads)
    else:
        partials = torch.full((ext.kv_attend_partials_floats(q_heads, d, splits),), float("nan"), device="cuda")
        ext.kv_rope_append_attend_split(qkv, cos_t, sin_t, *args, partials, position, d ** -0.5, q_heads, splits)
        merged = ext.kv_attend_merge(partials, q_heads, d, splits, torch.bfloat16)
    # what the step appended, and everything before it, is what FakeQuantCache's rule gives
    assert np.array_equal(codes_np(cache["k_codes"], bits), kq)
    assert np.array_equal(codes_np(cache["v_codes"], bits), vq)
    assert np.array_equal(to_np(cache["k_scale"]), ks) and np.array_equal(to_np(cache["v_scale"]), vs)
    got = to_np(merged).reshape(q_heads, d)
    assert rel_l2(got, want) <= 1e-2
    per_head = np.linalg.norm(got - want, axis=1) / np.linalg.norm(want, axis=1)
    assert per_head.max() <= 2e-2, per_head.argmax()  # no single head hides in the norm of the others

    if splits > 1:
        # o_proj over the oracle's attention output: heads of 64 padded to groups of 128, int8
        torch.manual_seed(3)
        n = 2048
        w = (torch.randn(n, q_heads * d) * 0.02).to(torch.bfloat16)
        canonical, scales = oracle.canonical_weight(to_np(w), 8, 128, d, None)
        res = torch.randn(1, n).to(torch.bfloat16)
        out = ext.wq_gemv_attn_merge(partials, splits, d, torch.from_numpy(canonical).cuda(),
                                     torch.from_numpy(scales).cuda(), 0, d, res.cuda(), torch.bfloat16)
        padded = oracle.pad_activation(want.reshape(1, -1), 128, d)
        exact = oracle.gemv_float64(padded, canonical, scales) + to_np(res).astype(np.float64)
        assert rel_l2(to_np(out), exact) <= 1e-2


@pytest.mark.parametrize("ctx,splits,t_max,q_heads,kv_heads,d", [
    (2048, 32, 4096, 32, 8, 64), (640, 32, 4096, 32, 8, 64), (0, 32, 4096, 32, 8, 64), (1, 32, 4096, 32, 8, 64),
    (63, 32, 4096, 32, 8, 64), (64, 32, 4096, 32, 8, 64), (65, 32, 4096, 32, 8, 64), (4094, 32, 4096, 32, 8, 64),
    (5002, 32, 5004, 32, 8, 64), (9000, 64, 9216, 32, 8, 64), (3000, 48, 4100, 8, 2, 64), (20000, 32, 20001, 16, 2, 64),
    (2048, 32, 4096, 32, 8, 128), (0, 32, 4096, 32, 8, 128), (65, 32, 4096, 32, 8, 128), (4094, 32, 4096, 32, 8, 128),
    (5002, 32, 5004, 32, 8, 128), (9000, 64, 9216, 8, 2, 128)])
@pytest.mark.parametrize("bits", [8, 4])
def test_long_cache_decode_step_on_the_matrix_core_against_the_oracle(ext, bits, ctx, splits, t_max, q_heads, kv_heads,
                                                                      d):
    """Caches of 4096 rows and more under grouped-query attention take the
    matrix-core form of the split step (codes as int8 operands, the query in three digits, the softmax weights
    in two): the same checks as the vector-ALU form gets, against the same oracle (appended codes and scales bit
    for bit, output rel-L2 <= 1e-2 and <= 2e-2 per head), at contexts around the 64-token slab boundaries, with
    one token and none, up to the cache's last row, with cache lengths that are not whole slabs. Rows beyond the
    position hold random codes and NaN scales: nothing of them may reach the result."""
    cache, qkv, cos_t, sin_t, want, (kq, ks, vq, vs) = decode_step_case(ext, bits, ctx, q_heads, kv_heads, d, seed=ctx,
                                                                        t_max=t_max)
    gen = torch.Generator(device="cuda").manual_seed(1)
    for name in ("k_codes", "v_codes"):
        cache[name][:, ctx + 1:] = torch.randint(0, 256, cache[name][:, ctx + 1:].shape, generator=gen,
                                                 device="cuda").to(torch.uint8).view(cache[name].dtype)
    for name in ("k_scale", "v_scale"):
        cache[name][:, ctx + 1:] = float("nan")
    position = torch.tensor([ctx], dtype=torch.int32, device="cuda")
    partials = torch.full((ext.kv_attend_partials_floats(q_heads, d, splits),), float("nan"), device="cuda")
    ext.kv_rope_append_attend_split(qkv, cos_t, sin_t, cache["k_codes"], cache["v_codes"], cache["k_scale"],
                                    cache["v_scale"], partials, position, d ** -0.5, q_heads, splits)
    merged = ext.kv_attend_merge(partials, q_heads, d, splits, torch.bfloat16)
    assert np.array_equal(codes_np(cache["k_codes"], bits)[:, : ctx + 1], kq)
    assert np.array_equal(codes_np(cache["v_codes"], bits)[:, : ctx + 1], vq)
    assert np.array_equal(to_np(cache["k_scale"])[:, : ctx + 1], ks)
    assert np.array_equal(to_np(cache["v_scale"])[:, : ctx + 1], vs)
    got = to_np(merged).reshape(q_heads, d)
    assert np.isfinite(got).all()
    assert rel_l2(got, want) <= 1e-2
    per_head = np.linalg.norm(got - want, axis=1) / np.linalg.norm(want, axis=1)
    assert per_head.max() <= 2e-2, per_head.argmax()
    print(f"int{bits} ctx {ctx} splits {splits} d {d}: rel-L2 {rel_l2(got, want):.2e}, worst head {per_head.max():.2e}")


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("tag,tol", [("f16", 2e-3), ("f32", 1e-3)])
@pytest.mark.parametrize("t_max,d", [(701, 64), (2304, 64), (2304, 128)])
def test_decode_step_attention_in_the_other_dtypes(ext, bits, tag, tol, t_max, d):
    """fp16 and fp32 models through the split step, on a cache short enough for the vector-ALU form (701 rows) and on
    one that takes the matrix-core form (2304 rows; heads of 64 and of 128), 700 cached tokens, against the oracle with
    that dtype's rounding points: the appended codes and scales bit for bit, the output within the dtype's share of
    the tolerance (fp32: what the kernels' own arithmetic leaves)."""
    q_heads, kv_heads, ctx, splits = 32, 8, 700, 8
    cache, qkv, cos_t, sin_t, want, (kq, ks, vq, vs) = decode_step_case(ext, bits, ctx, q_heads, kv_heads, d, seed=11,
                                                                        t_max=t_max, tag=tag)
    position = torch.tensor([ctx], dtype=torch.int32, device="cuda")
    partials = torch.full((ext.kv_attend_partials_floats(q_heads, d, splits),), float("nan"), device="cuda")
    ext.kv_rope_append_attend_split(qkv, cos_t, sin_t, cache["k_codes"], cache["v_codes"], cache["k_scale"],
                                    cache["v_scale"], partials, position, d ** -0.5, q_heads, splits)
    merged = ext.kv_attend_merge(partials, q_heads, d, splits, DTYPE_OF_TAG[tag])
    assert np.array_equal(codes_np(cache["k_codes"], bits)[:, : ctx + 1], kq)
    assert np.array_equal(codes_np(cache["v_codes"], bits)[:, : ctx + 1], vq)
    assert np.array_equal(to_np(cache["k_scale"])[:, : ctx + 1], ks)
    assert np.array_equal(to_np(cache["v_scale"])[:, : ctx + 1], vs)
    got = to_np(merged).reshape(q_heads, d)
    err = rel_l2(got, want)
    print(f"{tag} int{bits} cache of {t_max} rows, heads of {d}: rel-L2 {err:.2e}")
    assert err <= tol


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("ctx,t_max,splits,q_heads,kv_heads", [(0, 1, 8, 32, 8), (1, 2, 8, 32, 8), (63, 64, 8, 32, 8),
                                                            (64, 65, 8, 32, 8), (300, 301, 8, 32, 8), (300, 512, 32, 8, 2),
                                                            (700, 769, 16, 16, 4)])
def test_heads_of_128_take_the_matrix_core_form_on_short_caches_too(ext, bits, ctx, t_max, splits, q_heads, kv_heads):
    """With heads of 128 the entry point takes the matrix-core form of the split step whatever the cache's size (eight
    splits or more, four query heads per kv head): caches of one row, of exactly one slab and of a few hundred rows
    against the oracle, the checks of the long caches."""
    d = 128
    cache, qkv, cos_t, sin_t, want, (kq, ks, vq, vs) = decode_step_case(ext, bits, ctx, q_heads, kv_heads, d,
                                                                        seed=100 + ctx, t_max=t_max)
    for name in ("k_scale", "v_scale"):
        cache[name][:, ctx + 1:] = float("nan")
    position = torch.tensor([ctx], dtype=torch.int32, device="cuda")
    partials = torch.full((ext.kv_attend_partials_floats(q_heads, d, splits),), float("nan"), device="cuda")
    ext.kv_rope_append_attend_split(qkv, cos_t, sin_t, cache["k_codes"], cache["v_codes"], cache["k_scale"],
                                    cache["v_scale"], partials, position, d ** -0.5, q_heads, splits)
    merged = ext.kv_attend_merge(partials, q_heads, d, splits, torch.bfloat16)
    assert np.array_equal(codes_np(cache["k_codes"], bits)[:, : ctx + 1], kq)
    assert np.array_equal(codes_np(cache["v_codes"], bits)[:, : ctx + 1], vq)
    assert np.array_equal(to_np(cache["k_scale"])[:, : ctx + 1], ks)
    assert np.array_equal(to_np(cache["v_scale"])[:, : ctx + 1], vs)
    got = to_np(merged).reshape(q_heads, d)
    assert np.isfinite(got).all()
    assert rel_l2(got, want) <= 1e-2
    per_head = np.linalg.norm(got - want, axis=1) / np.linalg.norm(want, axis=1)
    assert per_head.max() <= 2e-2, per_head.argmax()
