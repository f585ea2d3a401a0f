#!/usr/bin/env python3
"""Writes regression_affine.npz beside this file from the C restatement in
oracle/: seeded bf16 weights (half N(0, 0.02), half adversarial groups), their
4- and 8-bit quantization, and float64 matmul results for a small seeded x.
Regression vectors only: they freeze the oracle, they are not evidence of
agreement with MLX (see README.md)."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from cases import adversarial_groups, seeded  # noqa: E402
from oracle import mlx_affine as o  # noqa: E402


def main():
    rows, K = 48, 256
    f = np.concatenate([
        seeded(7, 0, (rows // 2, K), 0.02),
        adversarial_groups(o, rows // 2 * K // 64, 64, seed=7).reshape(rows // 2, K),
    ])
    f = np.where(np.isfinite(f), f, np.float32(0)).astype(np.float32)
    f = np.clip(f, -1e3, 1e3)  # keeps the float64 matmul results well inside float32
    w = o.f32_to_bf16_bits(f)
    x = o.f32_to_bf16_bits(seeded(7, 1, (5, K), 1.0))
    out = {"w": w, "x": x}
    for bits in (4, 8):
        wq, s, b = o.c_quantize(w, o.BF16, 64, bits)
        out[f"wq{bits}"], out[f"scales{bits}"], out[f"biases{bits}"] = wq, s, b
        y = o.quantized_matmul_f64(o.bf16_bits_to_f32(x).astype(np.float64), wq, s, b, o.BF16, 64, bits)
        out[f"y{bits}"] = y.astype(np.float32)
    np.savez_compressed(os.path.join(HERE, "regression_affine.npz"), **out)
    print("wrote", os.path.join(HERE, "regression_affine.npz"))


if __name__ == "__main__":
    main()
