"""llmq_kv_decode_attention_static: the decode attention for callers that cannot allocate. Its partial
records and arrival counters live in a device array inside the library instead of a caller's workspace.
Called through the C ABI and compared bit for bit with llmq_kv_decode_attention on the same cache, on two
calls in a row of which the second is smaller (fewer heads, a shorter cache, another head width: its
records land where the first call's lay), and once more after the first shape again."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

DTYPE_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}
_WARMED = []   # non-empty once the entry point has run on the device


def make_case(ext, q_heads, kv_heads, d, t_max, length, bits, dtype, seed):
    gen = torch.Generator().manual_seed(seed)
    k = torch.randn(kv_heads, length, d, generator=gen).to(dtype).cuda()
    v = torch.randn(kv_heads, length, d, generator=gen).to(dtype).cuda()
    q = torch.randn(q_heads, d, generator=gen).to(dtype).cuda()
    width = d if bits == 8 else d // 2
    code_dtype = torch.int8 if bits == 8 else torch.uint8
    cache = dict(kc=torch.zeros(kv_heads, t_max, width, dtype=code_dtype, device="cuda"),
                 vc=torch.zeros(kv_heads, t_max, width, dtype=code_dtype, device="cuda"),
                 ks=torch.zeros(kv_heads, t_max, device="cuda"), vs=torch.zeros(kv_heads, t_max, device="cuda"))
    zero = torch.zeros(1, dtype=torch.int32, device="cuda")
    ext.kv_append(k, v, cache["kc"], cache["vc"], cache["ks"], cache["vs"], zero, False)
    return q, cache, torch.tensor([length], dtype=torch.int32, device="cuda")


def both_ways(lib, ext, q_heads, kv_heads, d, t_max, length, bits, dtype, seed):
    q, c, len_dev = make_case(ext, q_heads, kv_heads, d, t_max, length, bits, dtype, seed)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    scale = d ** -0.5
    floats = lib.llmq_kv_decode_workspace_floats(q_heads, d, t_max)
    workspace = torch.zeros(floats, device="cuda")
    want = torch.full((q_heads, d), float("nan"), dtype=dtype, device="cuda")
    got = torch.full((q_heads, d), float("nan"), dtype=dtype, device="cuda")
    tensors = (q.data_ptr(), c["kc"].data_ptr(), c["vc"].data_ptr(), c["ks"].data_ptr(), c["vs"].data_ptr())
    sizes = (q_heads, kv_heads, d, t_max, bits, DTYPE_CODE[dtype])
    rc = lib.llmq_kv_decode_attention(*tensors, want.data_ptr(), workspace.data_ptr(), len_dev.data_ptr(), scale,
                                      *sizes, stream)
    assert rc == 0, lib.llmq_last_error()
    torch.cuda.synchronize()
    free_before, reserved_before = torch.cuda.mem_get_info()[0], torch.cuda.memory_reserved()
    rc = lib.llmq_kv_decode_attention_static(*tensors, got.data_ptr(), len_dev.data_ptr(), scale, *sizes, stream)
    assert rc == 0, lib.llmq_last_error()
    torch.cuda.synchronize()
    if _WARMED:  # (the first call on the device may load the code object that holds the array)
        # the device's free memory (hipMemGetInfo) and torch's pool are what they were: the call allocated nothing
        assert torch.cuda.mem_get_info()[0] == free_before and torch.cuda.memory_reserved() == reserved_before
    _WARMED.append(True)
    assert torch.isfinite(want.float()).all()
    assert torch.equal(got.view(torch.int16 if dtype != torch.float32 else torch.int32),
                       want.view(torch.int16 if dtype != torch.float32 else torch.int32))
    return got


def test_static_scratch_attention_equals_the_workspace_form():
    from llmquant.hip import load_capi, load_extension

    lib, ext = load_capi(), load_extension()
    # Llama-3.2-1B geometry at a context of 2048 + 1: 33 splits x 32 heads of records
    both_ways(lib, ext, 32, 8, 64, 2049, 2049, 8, torch.bfloat16, seed=0)
    # a smaller call right after it: fewer heads and splits, wider heads, int4, another dtype
    both_ways(lib, ext, 8, 2, 128, 300, 211, 4, torch.float16, seed=1)
    # and a larger one again, fp32, a cache only partly filled
    both_ways(lib, ext, 32, 8, 128, 4096, 1000, 8, torch.float32, seed=2)
    both_ways(lib, ext, 4, 4, 64, 64, 1, 4, torch.bfloat16, seed=3)


def test_static_scratch_limits_are_errors():
    from llmquant.hip import load_capi

    lib = load_capi()
    one = ctypes.c_void_p(16)  # never dereferenced: the checks come first
    rc = lib.llmq_kv_decode_attention_static(one, one, one, one, one, one, one, 0.125, 256, 8, 64, 128, 8, 2, None)
    assert rc == 1 and b"up to 128 query heads" in lib.llmq_last_error()
    rc = lib.llmq_kv_decode_attention_static(one, one, one, one, one, one, one, 0.125, 32, 8, 96, 128, 8, 2, None)
    assert rc == 1 and b"head_dim" in lib.llmq_last_error()
    rc = lib.llmq_kv_decode_attention_static(None, one, one, one, one, one, one, 0.125, 32, 8, 64, 128, 8, 2, None)
    assert rc == 1 and b"null tensor pointer" in lib.llmq_last_error()


def test_static_scratch_call_replays_from_a_graph():
    """The call allocates nothing and records no memset, so it can be captured: every replay, with fresh
    queries and eager calls between the replays, equals the eager workspace form."""
    from llmquant.hip import load_capi, load_extension

    lib, ext = load_capi(), load_extension()
    q_heads, kv_heads, d, t_max, length = 32, 8, 64, 1024, 700
    q, c, len_dev = make_case(ext, q_heads, kv_heads, d, t_max, length, 8, torch.bfloat16, seed=5)
    out = torch.zeros(q_heads, d, dtype=torch.bfloat16, device="cuda")
    tensors = (q.data_ptr(), c["kc"].data_ptr(), c["vc"].data_ptr(), c["ks"].data_ptr(), c["vs"].data_ptr())
    sizes = (q_heads, kv_heads, d, t_max, 8, 2)

    def call():
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc = lib.llmq_kv_decode_attention_static(*tensors, out.data_ptr(), len_dev.data_ptr(), d ** -0.5, *sizes, stream)
        assert rc == 0, lib.llmq_last_error()

    call()  # the first call on the device looks the array's address up: not inside a capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    ws = torch.zeros(ext.kv_decode_workspace_floats(q_heads, d, t_max), device="cuda")
    for replay in range(4):
        q.normal_()
        len_dev.fill_(length - 100 * replay)
        want = ext.kv_decode_attention(q, c["kc"], c["vc"], c["ks"], c["vs"], ws, len_dev, d ** -0.5)
        both_ways(lib, ext, 8, 2, 128, 300, 211, 4, torch.float16, seed=replay)  # eager work on the shared array
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), replay
