"""Seeded and adversarial inputs shared by the CPU (oracle) tests and the GPU
parity tests.  numpy only: importable without torch or a device."""
import json
import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def seeded(config: int, tensor: int, shape, std: float) -> np.ndarray:
    """Synthetic input convention: numpy default_rng(1000*config + tensor),
    float32 normal scaled by std."""
    rng = np.random.default_rng(1000 * config + tensor)
    return (rng.standard_normal(shape, dtype=np.float32) * np.float32(std)).astype(np.float32)


def adversarial_groups(o, n_groups: int, gs: int, seed: int) -> np.ndarray:
    """float32 rows of groups built to hit the corners of the algorithm:
    ties at x.5 code boundaries, all-equal groups, zeros of both signs, tiny
    values under the eps clamp, denormals, a huge dynamic range, max-only and
    min-only edges."""
    rng = np.random.default_rng(seed)
    g = np.empty((n_groups, gs), dtype=np.float32)
    for i in range(n_groups):
        kind = i % 12
        if kind == 0:   # exact grid: codes land on integers and on .5 ties
            step = np.float32(2.0 ** rng.integers(-12, 4))
            g[i] = rng.integers(-15, 16, gs).astype(np.float32) * step * np.float32(0.5)
        elif kind == 1:  # all equal
            g[i] = np.float32(rng.standard_normal() * 0.02)
        elif kind == 2:  # zeros of both signs
            g[i] = np.where(rng.random(gs) < 0.5, np.float32(0.0), np.float32(-0.0))
        elif kind == 3:  # below the eps clamp
            g[i] = rng.standard_normal(gs).astype(np.float32) * np.float32(1e-8)
        elif kind == 4:  # float32 denormals (flush to zero in bf16 inputs, kept for f32)
            g[i] = rng.standard_normal(gs).astype(np.float32) * np.float32(1e-40)
        elif kind == 5:  # huge dynamic range
            g[i] = rng.standard_normal(gs).astype(np.float32) * np.float32(10.0) ** rng.integers(-6, 6, gs).astype(np.float32)
        elif kind == 6:  # all positive: the maximum is the edge
            g[i] = np.abs(rng.standard_normal(gs)).astype(np.float32)
        elif kind == 7:  # all negative: the minimum is the edge
            g[i] = -np.abs(rng.standard_normal(gs)).astype(np.float32)
        elif kind == 8:  # |min| == |max|
            v = rng.standard_normal(gs).astype(np.float32)
            v[0], v[1] = np.float32(-3.0), np.float32(3.0)
            g[i] = np.clip(v, -3, 3)
        elif kind == 9:  # one outlier
            v = rng.standard_normal(gs).astype(np.float32) * np.float32(0.01)
            v[rng.integers(gs)] = np.float32(50.0)
            g[i] = v
        elif kind == 10:  # large magnitudes
            g[i] = rng.standard_normal(gs).astype(np.float32) * np.float32(1e30)
        else:
            g[i] = rng.standard_normal(gs).astype(np.float32) * np.float32(0.02)
    return g


def storage(o, f32: np.ndarray, dtype: int) -> np.ndarray:
    if dtype == o.BF16:
        return o.f32_to_bf16_bits(f32)
    if dtype == o.F16:
        with np.errstate(over="ignore"):
            h = np.clip(f32, -60000, 60000).astype(np.float16)
        return h.view(np.uint16)
    return f32


def pack_codes(codes: np.ndarray, bits: int) -> np.ndarray:
    """codes [..., n] -> uint32 words [..., n*bits/32], element i of a word in
    bits [i*bits, (i+1)*bits).  Plain Python loops: an independent statement of
    the layout, not the oracle's vectorised one."""
    per = 32 // bits
    flat = np.asarray(codes, dtype=np.uint64).reshape(-1, per)
    words = np.zeros(flat.shape[0], dtype=np.uint64)
    for i in range(per):
        words |= flat[:, i] << np.uint64(i * bits)
    return words.astype(np.uint32).reshape(*np.shape(codes)[:-1], np.shape(codes)[-1] // per)


def known_answers():
    """The hand-computed cases of golden/kat_affine.json as
    (name, bits, float32 group[64], words uint32, scale bits, bias bits)."""
    with open(os.path.join(GOLDEN, "kat_affine.json")) as f:
        spec = json.load(f)
    out = []
    for case in spec["cases"]:
        g = case["group"]
        codes = None
        if "ramp16_over_16" in g:
            r = g["ramp16_over_16"]
            vals = np.tile(np.arange(r["first"], r["last"] + 1, dtype=np.float32) / np.float32(16), r["repeat"])
        elif "codes_over_256_minus_half" in g:
            codes = np.array(g["codes_over_256_minus_half"], dtype=np.uint32)
            vals = codes.astype(np.float32) / np.float32(256) - np.float32(0.5)
        else:
            vals = np.full(64, g["constant"], dtype=np.float32)
        for idx, v in g.get("override", {}).items():
            vals[int(idx)] = np.float32(v)
        assert vals.shape == (64,)
        if case["words"] == "pack_codes_little_end_first":
            words = pack_codes(codes, case["bits"])
        else:
            words = np.array([int(w, 16) for w in case["words"]], dtype=np.uint32)
        out.append((case["name"], case["bits"], vals, words, int(case["scale_bits"], 16), int(case["bias_bits"], 16)))
    return out
