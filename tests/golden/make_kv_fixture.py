"""Writes tests/golden/kv_case.npz: a small seeded KV-cache case with the codes, scales and
attention output the CPU oracle gives for it. Run from the repository root:

    python tests/golden/make_kv_fixture.py

The oracle functions used here are pinned by tests/test_oracle_quant.py first; the fixture then
lets the GPU tests compare against stored bytes.
"""

import pathlib
import sys

import numpy as np

ROOT = pathlib.Path(__file__).resolve().parent.parent.parent
sys.path.insert(0, str(ROOT / "oracle"))
import llmq_oracle as oracle  # noqa: E402


def main():
    rng = np.random.default_rng(20240)
    kv_heads, q_heads, t, d = 2, 8, 37, 64
    channel = np.exp(0.5 * rng.standard_normal(d)).astype(np.float32)  # RoPE-like per-channel spread
    k = oracle.round_to((rng.standard_normal((kv_heads, t, d)) * channel).astype(np.float32), "bf16")
    v = oracle.round_to((rng.standard_normal((kv_heads, t, d)) * channel).astype(np.float32), "bf16")
    q = oracle.round_to(rng.standard_normal((q_heads, d)).astype(np.float32), "bf16")
    out = {"k": oracle.bf16_bits(k).reshape(k.shape), "v": oracle.bf16_bits(v).reshape(v.shape),
           "q": oracle.bf16_bits(q).reshape(q.shape)}
    for bits in (8, 4):
        kc, ks = oracle.kv_quant(k, bits)
        vc, vs = oracle.kv_quant(v, bits)
        attn = oracle.gqa_decode_attention(q, oracle.kv_dequant(kc, ks, "bf16"), oracle.kv_dequant(vc, vs, "bf16"),
                                           d ** -0.5, "f32")
        out.update({f"k_codes{bits}": kc, f"v_codes{bits}": vc, f"k_scale{bits}": ks, f"v_scale{bits}": vs,
                    f"attn{bits}": attn})
    np.savez_compressed(ROOT / "tests" / "golden" / "kv_case.npz", **out)


if __name__ == "__main__":
    main()
