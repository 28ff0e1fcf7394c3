"""Writes the small golden vectors under tests/golden/ from the CPU oracle (oracle/rope_oracle.c).

The reference stores no vectors of its own for this path (its checks are computed on the fly,
test.py:230, example_llmc_rope.cu:286), so these are made from the C restatement after it has
been pinned by tests/test_oracle.py.  Inputs are seeded; running this script again must
reproduce the committed files bit for bit (tests/test_golden.py checks that).

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import oracle as O  # noqa: E402

CASES = {
    # name: (B, T, Nq, Nkv, HS, theta, use_scaled, dtype, layout)
    "rope_fp32_qkv_tiny": (1, 4, 2, 2, 8, 10000.0, False, "fp32", "qkv"),
    "rope_fp32_qkv_gqa": (2, 6, 4, 1, 16, 500000.0, False, "fp32", "qkv"),
    "rope_fp32_qkv_scaled": (1, 8, 2, 2, 64, 10000.0, True, "fp32", "qkv"),
    "rope_fp32_heads_gpt2": (1, 5, 12, 0, 64, 10000.0, False, "fp32", "heads"),
    "rope_bf16_heads_llama3": (1, 7, 8, 0, 128, 500000.0, False, "bf16", "heads"),
    # the half-split pair layout (element i pairs with element i + HS/2), every head rotated
    "rope_half_fp32_heads": (2, 5, 3, 0, 32, 10000.0, False, "fp32", "half"),
    "rope_half_bf16_heads_llama3": (1, 6, 8, 0, 128, 500000.0, False, "bf16", "half"),
}


def make(name):
    B, T, Nq, Nkv, HS, theta, scaled, dtype, layout = CASES[name]
    rng = np.random.default_rng(sum(map(ord, name)))
    heads = Nq + 2 * Nkv if layout == "qkv" else Nq
    x = rng.standard_normal((B, T, heads, HS)).astype(np.float32)
    freqs = O.freqs_cis(HS, T, theta, scaled)
    out = {"freqs": freqs, "shape": np.array([B, T, Nq, Nkv, HS], dtype=np.int64)}
    if dtype == "fp32":
        out["x"] = x
        if layout == "qkv":
            out["y"] = O.rope_forward_qkv_f32(x, freqs, Nq, Nkv)
            out["dx"] = O.rope_backward_qkv_f32(out["y"], freqs, Nq, Nkv)
        elif layout == "half":
            out["y"] = O.rope_half_forward_heads_f32(x, freqs)
            out["dx"] = O.rope_half_backward_heads_f32(out["y"], freqs)
        else:
            out["y"] = O.rope_forward_heads_f32(x, freqs)
            out["dx"] = O.rope_backward_heads_f32(out["y"], freqs)
    else:
        xb = O.f32_to_bf16(x)
        out["x"] = xb
        out["y"] = O.rope_half_forward_heads_bf16(xb, freqs) if layout == "half" else O.rope_forward_heads_bf16(xb, freqs)
    return out


def scale_bias_case():
    rng = np.random.default_rng(20)
    x = O.f32_to_bf16(rng.standard_normal(2048).astype(np.float32) * 4)
    return {"x": x, "scale": np.float32(0.75), "bias": np.float32(-1.25),
            "y": O.scale_bias_bf16(x, 0.75, -1.25)}


def main():
    for name in CASES:
        np.savez(os.path.join(HERE, name + ".npz"), **make(name))
    np.savez(os.path.join(HERE, "scale_bias_bf16.npz"), **scale_bias_case())
    print("wrote", len(CASES) + 1, "files to", HERE)


if __name__ == "__main__":
    main()
