"""CPU tests that pin the oracle (oracle/mlx_affine.{c,py}) before anything is
compared against it: hand-computed known answers, invariants the algorithm
fixes, brute force on tiny cases, the two restatements against each other, and
the matmul against float64 numpy."""
import os

import numpy as np
import pytest

from cases import GOLDEN, adversarial_groups, known_answers, pack_codes, seeded, storage


# ---------------------------------------------------------------------------
# quantize: known answers
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("impl", ["c", "numpy"])
@pytest.mark.parametrize("case", known_answers(), ids=lambda c: c[0])
def test_known_answers(oracle, impl, case):
    o = oracle
    name, bits, vals, words, scale_bits, bias_bits = case
    w = o.f32_to_bf16_bits(vals).reshape(1, 64)
    assert np.array_equal(o.bf16_bits_to_f32(w).reshape(-1), vals), "case values must be exact in bf16"
    fn = o.c_quantize if impl == "c" else o.quantize
    wq, s, b = fn(w, o.BF16, 64, bits)
    assert [hex(v) for v in wq.reshape(-1)] == [hex(v) for v in words]
    assert hex(int(s.reshape(-1)[0])) == hex(scale_bits)
    assert hex(int(b.reshape(-1)[0])) == hex(bias_bits)


@pytest.mark.parametrize("impl", ["c", "numpy"])
def test_known_answers_3_5_6_bits(oracle, impl):
    """Byte packs of the odd widths, from closed forms worked out by hand
    (tests/golden/README.md): a ramp that quantizes to codes 0, 1, 2, ... in
    order, so pack j is a known integer written little-end first."""
    o = oracle
    fn = o.c_quantize if impl == "c" else o.quantize
    # 3 bits: values (i-4)/8, codes 0..7 eight times; each 3-byte pack is 0xFAC688
    vals = np.tile((np.arange(8, dtype=np.float32) - 4) / np.float32(8), 8)
    wq, s, b = fn(o.f32_to_bf16_bits(vals).reshape(1, 64), o.BF16, 64, 3)
    assert wq.shape == (1, 6) and s[0, 0] == 0x3E00 and b[0, 0] == 0xBF00
    assert wq.view(np.uint8).reshape(-1).tolist() == [0x88, 0xC6, 0xFA] * 8
    assert [hex(v) for v in wq.reshape(-1)[:3]] == ["0x88fac688", "0xc688fac6", "0xfac688fa"]
    # 6 bits: values (i-32)/64, codes 0..63; pack j (4 codes, 3 bytes) = 0x0C2040 + j*0x104104
    vals = (np.arange(64, dtype=np.float32) - 32) / np.float32(64)
    wq, s, b = fn(o.f32_to_bf16_bits(vals).reshape(1, 64), o.BF16, 64, 6)
    assert wq.shape == (1, 12) and s[0, 0] == 0x3C80 and b[0, 0] == 0xBF00
    expect = []
    for j in range(16):
        v = 0x0C2040 + j * 0x104104
        expect += [v & 0xFF, (v >> 8) & 0xFF, (v >> 16) & 0xFF]
    assert wq.view(np.uint8).reshape(-1).tolist() == expect
    # 5 bits: values (i-16)/32, codes 0..31 twice; pack j (8 codes, 5 bytes) = P0 + (j%4)*8*R,
    # P0 = sum k*32^k (k<8), R = (32^8-1)/31
    vals = np.tile((np.arange(32, dtype=np.float32) - 16) / np.float32(32), 2)
    wq, s, b = fn(o.f32_to_bf16_bits(vals).reshape(1, 64), o.BF16, 64, 5)
    assert wq.shape == (1, 10) and s[0, 0] == 0x3D00 and b[0, 0] == 0xBF00
    p0, r = sum(k * 32 ** k for k in range(8)), (32 ** 8 - 1) // 31
    assert (p0, r) == (0x398A418820, 0x842108421)
    expect = []
    for j in range(8):
        v = p0 + (j % 4) * 8 * r
        expect += [(v >> (8 * i)) & 0xFF for i in range(5)]
    assert wq.view(np.uint8).reshape(-1).tolist() == expect


@pytest.mark.parametrize("bits", [3, 5, 6])
def test_odd_widths_restatements_agree_and_round_trip(oracle, bits):
    o = oracle
    n_bins = (1 << bits) - 1
    for gs in (32, 64, 128):
        w = o.f32_to_bf16_bits(seeded(9, 70 + bits, (32, 512), 0.02))
        c, n = o.c_quantize(w, o.BF16, gs, bits), o.quantize(w, o.BF16, gs, bits)
        assert c[0].shape == (32, 512 * bits // 32)
        for a, b in zip(c, n):
            assert np.array_equal(a, b)
        codes = o.unpack_codes(c[0], bits)
        assert codes.shape == (32, 512) and codes.max() == n_bins
        assert np.array_equal(pack_stream(codes, bits), c[0])
        assert np.array_equal(o.c_dequantize_f64(*c, o.BF16, gs, bits), o.dequantize_exact(*c, o.BF16, gs, bits))
        err = np.abs(o.dequantize_exact(*c, o.BF16, gs, bits) - o.bf16_bits_to_f32(w))
        step = np.repeat(np.abs(o.bf16_bits_to_f32(c[1])), gs, axis=1)
        assert (err <= step * (1.0 + n_bins * 2.0 ** -9) + 1e-12).all()


def pack_stream(codes, bits):
    """Independent loop-based statement of the bit stream: python integers."""
    out = []
    for row in codes:
        v = 0
        for i, c in enumerate(row):
            v |= int(c) << (i * bits)
        out.append([(v >> (32 * j)) & 0xFFFFFFFF for j in range(len(row) * bits // 32)])
    return np.array(out, dtype=np.uint32)


def test_known_answers_as_float32_and_float16(oracle):
    """The same groups are exact in float16/float32, and the answers do not
    depend on the storage type beyond the final cast of scale and bias."""
    o = oracle
    for name, bits, vals, words, scale_bits, bias_bits in known_answers():
        wq32, s32, b32 = o.c_quantize(vals.reshape(1, 64), o.F32, 64, bits)
        assert np.array_equal(wq32.reshape(-1), words), name
        assert o.f32_to_bf16_bits(s32).reshape(-1)[0] == scale_bits, name
        assert o.f32_to_bf16_bits(b32).reshape(-1)[0] == bias_bits, name
        h = vals.astype(np.float16).view(np.uint16).reshape(1, 64)
        wq16, _, b16 = o.c_quantize(h, o.F16, 64, bits)
        assert np.array_equal(wq16.reshape(-1), words), name
        assert b16.view(np.float16).reshape(-1)[0] == np.float16(o.bf16_bits_to_f32(np.uint16(bias_bits))), name


# ---------------------------------------------------------------------------
# quantize: the two restatements agree bit for bit
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("gs", [32, 64, 128])
@pytest.mark.parametrize("dtype_name", ["bf16", "f16", "f32"])
def test_c_and_numpy_restatements_agree(oracle, bits, gs, dtype_name):
    o = oracle
    dtype = {"bf16": o.BF16, "f16": o.F16, "f32": o.F32}[dtype_name]
    rows, K = 64, 1024
    for f32 in (seeded(9, bits * 1000 + gs, (rows, K), 0.02),
                adversarial_groups(o, rows * K // gs, gs, seed=bits + gs).reshape(rows, K)):
        w = storage(o, f32, dtype)
        c = o.c_quantize(w, dtype, gs, bits)
        n = o.quantize(w, dtype, gs, bits)
        for what, a, b in zip(("wq", "scales", "biases"), c, n):
            assert a.dtype == b.dtype and a.shape == b.shape, what
            assert np.array_equal(a, b), what


# ---------------------------------------------------------------------------
# quantize: brute force with Python's own floats (float64 arithmetic rounded to
# float32 after every operation is float32 arithmetic for + - * / on float32
# inputs, since 53 >= 2*24 + 2)
# ---------------------------------------------------------------------------
def _f32(v):
    return float(np.float32(v))


def _rne(v: float) -> float:
    return float(round(v))  # Python's round() is round-half-to-even


def _brute_group(vals, bits):
    n_bins = float((1 << bits) - 1)
    w_min, w_max = min(vals), max(vals)
    mask = abs(w_min) > abs(w_max)
    scale = max(_f32((_f32(w_max - w_min)) / n_bins), _f32(1e-7))
    scale = scale if mask else -scale
    edge = w_min if mask else w_max
    q0 = _rne(_f32(edge / scale))
    bias = 0.0
    if q0 != 0:
        scale = _f32(edge / q0)
        bias = edge
    codes = []
    for e in vals:
        q = _rne(_f32(_f32(e - bias) / scale))
        codes.append(int(min(max(q, 0.0), n_bins)))
    return codes, scale, bias


@pytest.mark.parametrize("bits", [4, 8])
def test_brute_force_python_floats(oracle, bits):
    o = oracle
    rng = np.random.default_rng(42 + bits)
    f32 = np.concatenate([
        rng.standard_normal((40, 32), dtype=np.float32) * np.float32(0.02),
        adversarial_groups(o, 48, 32, seed=3)[np.isfinite(adversarial_groups(o, 48, 32, seed=3)).all(axis=1)],
    ])
    w = o.f32_to_bf16_bits(f32)
    vals = o.bf16_bits_to_f32(w)
    wq, s, b = o.c_quantize(w, o.BF16, 32, bits)
    got_codes = o.unpack_codes(wq, bits)
    for g in range(vals.shape[0]):
        codes, scale, bias = _brute_group([float(v) for v in vals[g]], bits)
        assert list(got_codes[g]) == codes, g
        assert s[g, 0] == o.f32_to_bf16_bits(np.float32(scale)), g
        assert b[g, 0] == o.f32_to_bf16_bits(np.float32(bias)), g


# ---------------------------------------------------------------------------
# quantize: invariants
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("bits", [4, 8])
def test_invariants(oracle, bits):
    o = oracle
    gs = 64
    n_bins = (1 << bits) - 1
    w = o.f32_to_bf16_bits(seeded(9, 11 + bits, (256, 512), 0.02))
    f = o.bf16_bits_to_f32(w).reshape(-1, gs)
    wq, s, b = o.c_quantize(w, o.BF16, gs, bits)
    assert wq.shape == (256, 512 * bits // 32) and s.shape == b.shape == (256, 512 // gs)
    codes = o.unpack_codes(wq, bits).reshape(-1, gs)
    sf = o.bf16_bits_to_f32(s).reshape(-1)
    bf = o.bf16_bits_to_f32(b).reshape(-1)
    assert codes.max() <= n_bins
    w_min, w_max = f.min(axis=1), f.max(axis=1)
    mask = np.abs(w_min) > np.abs(w_max)
    # the sign of the scale says which end is the edge; the bias IS the edge
    # element (a bf16 value, so the cast does not move it) and its code is 0
    assert np.array_equal(sf > 0, mask)
    edge = np.where(mask, w_min, w_max)
    assert np.array_equal(bf, edge)
    edge_pos = np.where(mask, f.argmin(axis=1), f.argmax(axis=1))
    assert (codes[np.arange(len(codes)), edge_pos] == 0).all()
    # the far end reaches the top code or the one below it (the re-fitted scale
    # moves by less than 1/(2*q0) relatively)
    far_pos = np.where(mask, f.argmax(axis=1), f.argmin(axis=1))
    assert (codes[np.arange(len(codes)), far_pos] >= n_bins - 1).all()
    # reconstruction error: half a step of the float32 scale, plus what the
    # bf16 rounding of the scale adds at the far end (n_bins * 2^-9 steps)
    deq = codes.astype(np.float64) * sf[:, None].astype(np.float64) + bf[:, None].astype(np.float64)
    err = np.abs(deq - f.astype(np.float64))
    step = np.abs(sf)[:, None].astype(np.float64)
    assert (err <= step * (1.0 + n_bins * 2.0 ** -9) + 1e-12).all()
    assert (err <= step * (0.5 + n_bins * 2.0 ** -9) + 1e-12).mean() > 0.99


def test_negation_symmetry(oracle):
    """quantize(-w) has the same codes, and scale and bias negated: negation
    swaps min and max and every float32 operation used is odd-symmetric
    (rint ties to even included).  Groups with |min| == |max| are excluded
    (the strict comparison picks the maximum for both signs)."""
    o = oracle
    w = o.f32_to_bf16_bits(seeded(9, 21, (64, 1024), 0.02))
    neg = w ^ np.uint16(0x8000)
    for bits in (4, 8):
        wq, s, b = o.c_quantize(w, o.BF16, 64, bits)
        wq_n, s_n, b_n = o.c_quantize(neg, o.BF16, 64, bits)
        f = o.bf16_bits_to_f32(w).reshape(-1, 64)
        ok = (np.abs(f.min(axis=1)) != np.abs(f.max(axis=1))).reshape(s.shape)
        per_group_words = 64 * bits // 32
        okw = np.repeat(ok, per_group_words, axis=1)
        assert np.array_equal(wq[okw], wq_n[okw])
        assert np.array_equal(s[ok] ^ np.uint16(0x8000), s_n[ok])
        nz = (b[ok] & 0x7FFF) != 0
        assert np.array_equal((b[ok] ^ np.uint16(0x8000))[nz], b_n[ok][nz])


def test_power_of_two_scaling(oracle):
    """Scaling a group by 2^k scales scale and bias by 2^k and keeps the codes
    (every operation commutes with an exact power-of-two factor while nothing
    underflows and the eps clamp is not active)."""
    o = oracle
    f = seeded(9, 31, (32, 512), 0.02)
    w = o.f32_to_bf16_bits(f)
    w8 = o.f32_to_bf16_bits(o.bf16_bits_to_f32(w) * np.float32(8.0))
    for bits in (4, 8):
        wq, s, b = o.c_quantize(w, o.BF16, 64, bits)
        wq8, s8, b8 = o.c_quantize(w8, o.BF16, 64, bits)
        assert np.array_equal(wq, wq8)
        assert np.array_equal(o.bf16_bits_to_f32(s) * np.float32(8), o.bf16_bits_to_f32(s8))
        assert np.array_equal(o.bf16_bits_to_f32(b) * np.float32(8), o.bf16_bits_to_f32(b8))


@pytest.mark.parametrize("bits", [4, 8])
def test_exact_grid_round_trip(oracle, bits):
    """Weights that already lie on a grid code*step + bias, with both end codes
    present and step a power of two, come back with exactly those codes."""
    o = oracle
    rng = np.random.default_rng(5 + bits)
    n_bins = (1 << bits) - 1
    codes = rng.integers(0, n_bins + 1, (128, 64)).astype(np.uint32)
    codes[:, 0], codes[:, 1] = 0, n_bins
    # min edge: |bias| must exceed |bias + n_bins*step|: bias = -(n_bins+1)/2*step
    step = np.float32(2.0 ** -10)
    bias = np.float32(-(n_bins + 1) / 2) * step
    f = codes.astype(np.float32) * step + bias
    w = o.f32_to_bf16_bits(f)
    assert np.array_equal(o.bf16_bits_to_f32(w), f)
    wq, s, b = o.c_quantize(w.reshape(128, 64), o.BF16, 64, bits)
    assert np.array_equal(o.unpack_codes(wq, bits), codes)
    assert (o.bf16_bits_to_f32(s) == step).all() and (o.bf16_bits_to_f32(b) == bias).all()
    # and dequantize inverts it exactly
    d = o.c_dequantize(wq, s, b, o.BF16, 64, bits)
    assert np.array_equal(d, w.reshape(128, 64))


def test_packing_layout(oracle):
    """unpack_codes and the C quantizer agree with an independent loop-based
    packer on where element i of a word lives."""
    o = oracle
    rng = np.random.default_rng(8)
    for bits in (4, 8):
        codes = rng.integers(0, 1 << bits, (7, 128)).astype(np.uint32)
        words = pack_codes(codes, bits)
        assert np.array_equal(o.unpack_codes(words, bits), codes)
    assert pack_codes(np.arange(8, dtype=np.uint32)[None], 4)[0, 0] == 0x76543210
    assert pack_codes(np.array([[0x11, 0x22, 0x33, 0x44]], dtype=np.uint32), 8)[0, 0] == 0x44332211


def test_argument_errors(oracle):
    o = oracle
    w = np.zeros((4, 96), dtype=np.uint16)
    with pytest.raises(ValueError):
        o.quantize(w, o.BF16, 64, 4)  # 96 % 64
    with pytest.raises(ValueError):
        o.c_quantize(w, o.BF16, 64, 4)
    with pytest.raises(ValueError):
        o.quantize(np.zeros((64,), dtype=np.uint16), o.BF16, 64, 4)  # ndim < 2
    with pytest.raises(ValueError):
        o.quantize(np.zeros((4, 128), dtype=np.uint16), o.BF16, 48, 4)
    with pytest.raises(ValueError):
        o.c_quantize(np.zeros((4, 128), dtype=np.uint16), o.BF16, 64, 7)


# ---------------------------------------------------------------------------
# dequantize and matmul
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("bits", [4, 8])
def test_dequantize_definitions(oracle, bits):
    o = oracle
    w = o.f32_to_bf16_bits(seeded(9, 41, (32, 512), 0.02))
    wq, s, b = o.c_quantize(w, o.BF16, 64, bits)
    exact = o.dequantize_exact(wq, s, b, o.BF16, 64, bits)
    # independent statement of q*s+b with python loops on a few rows
    codes = o.unpack_codes(wq, bits)
    sf, bf = o.bf16_bits_to_f32(s), o.bf16_bits_to_f32(b)
    for n in (0, 13, 31):
        for k in (0, 1, 63, 64, 200, 511):
            assert exact[n, k] == float(codes[n, k]) * float(sf[n, k // 64]) + float(bf[n, k // 64])
    assert np.array_equal(o.c_dequantize_f64(wq, s, b, o.BF16, 64, bits), exact)
    # storage-type dequantize (two roundings) agrees between the restatements
    assert np.array_equal(o.c_dequantize(wq, s, b, o.BF16, 64, bits), o.dequantize(wq, s, b, o.BF16, 64, bits))


@pytest.mark.parametrize("bits,gs", [(4, 64), (8, 64), (4, 32), (8, 128)])
def test_qmm_against_float64_matmul(oracle, bits, gs):
    """The C qmm_t (float32 accumulation) is a textbook product: it matches
    float64 numpy on the exactly dequantized weights to float32 round-off."""
    o = oracle
    M, K, N = 9, 512, 96
    x = o.f32_to_bf16_bits(seeded(8, 0, (M, K), 1.0))
    w = o.f32_to_bf16_bits(seeded(8, 1, (N, K), 0.02))
    bias = o.f32_to_bf16_bits(seeded(8, 2, (N,), 0.02))
    wq, s, b = o.c_quantize(w, o.BF16, gs, bits)
    x64 = o.bf16_bits_to_f32(x).astype(np.float64)
    ref = o.quantized_matmul_f64(x64, wq, s, b, o.BF16, gs, bits)
    # float64 reference restated as an explicit loop over groups (factorised form)
    codes = o.unpack_codes(wq, bits).astype(np.float64)
    sf, bf = o.bf16_bits_to_f32(s).astype(np.float64), o.bf16_bits_to_f32(b).astype(np.float64)
    fact = np.zeros((M, N))
    for g in range(K // gs):
        xs = x64[:, g * gs:(g + 1) * gs]
        fact += (xs @ codes[:, g * gs:(g + 1) * gs].T) * sf[:, g] + xs.sum(axis=1, keepdims=True) * bf[:, g]
    assert np.allclose(fact, ref, rtol=1e-12, atol=1e-12)
    y32 = o.c_qmm_t(x, o.BF16, wq, s, b, o.BF16, None, gs, bits, y_dtype=o.F32, threads=2)
    assert np.abs(y32 - ref).max() <= 1e-5 * np.abs(ref).max() + 1e-6
    y16 = o.c_qmm_t(x, o.BF16, wq, s, b, o.BF16, bias, gs, bits, threads=1)
    ref_b = ref + o.bf16_bits_to_f32(bias).astype(np.float64)
    err = np.abs(o.bf16_bits_to_f32(y16).astype(np.float64) - ref_b).max(axis=1) / np.abs(ref_b).max(axis=1)
    assert err.max() <= 1e-2


def test_qmm_one_hot_and_ones(oracle):
    """One-hot rows of x return dequantized weight columns; a row of ones
    returns row sums: pins the k <-> (word, nibble) mapping end to end."""
    o = oracle
    K, N = 128, 40
    w = o.f32_to_bf16_bits(seeded(8, 5, (N, K), 0.02))
    for bits in (4, 8):
        wq, s, b = o.c_quantize(w, o.BF16, 64, bits)
        deq = o.dequantize_exact(wq, s, b, o.BF16, 64, bits)
        x = np.eye(K, dtype=np.float32)
        y = o.c_qmm_t(o.f32_to_bf16_bits(x), o.BF16, wq, s, b, o.BF16, None, 64, bits, y_dtype=o.F32)
        assert np.array_equal(y, deq.T.astype(np.float32))
        ones = o.f32_to_bf16_bits(np.ones((1, K), dtype=np.float32))
        y1 = o.c_qmm_t(ones, o.BF16, wq, s, b, o.BF16, None, 64, bits, y_dtype=o.F32)
        assert np.allclose(y1[0], deq.sum(axis=1), rtol=1e-5, atol=1e-6)


def test_storage_type_accumulation_is_not_a_parity_target(oracle):
    """Documents why the matmul oracle is exact math: a running sum kept in
    bf16 (MLX's generic CPU loop on x86) strays from the exact result by more
    than the 1e-2 * row-max budget at K = 3072."""
    o = oracle
    M, K, N = 4, 3072, 64
    x = o.f32_to_bf16_bits(seeded(8, 7, (M, K), 1.0))
    w = o.f32_to_bf16_bits(seeded(8, 8, (N, K), 0.02))
    wq, s, b = o.c_quantize(w, o.BF16, 64, 4)
    ref = o.quantized_matmul_f64(o.bf16_bits_to_f32(x).astype(np.float64), wq, s, b, o.BF16, 64, 4)
    y = o.c_qmm_t(x, o.BF16, wq, s, b, o.BF16, None, 64, 4, accumulate="storage")
    err = np.abs(o.bf16_bits_to_f32(y).astype(np.float64) - ref).max(axis=1) / np.abs(ref).max(axis=1)
    assert err.max() > 1e-2


# ---------------------------------------------------------------------------
# regression fixture
# ---------------------------------------------------------------------------
def test_regression_fixture(oracle):
    o = oracle
    path = os.path.join(GOLDEN, "regression_affine.npz")
    data = np.load(path, allow_pickle=False)
    for bits in (4, 8):
        w = data["w"]
        for impl in (o.c_quantize, o.quantize):
            wq, s, b = impl(w, o.BF16, 64, bits)
            assert np.array_equal(wq, data[f"wq{bits}"])
            assert np.array_equal(s, data[f"scales{bits}"])
            assert np.array_equal(b, data[f"biases{bits}"])
        y = o.c_qmm_t(data["x"], o.BF16, data[f"wq{bits}"], data[f"scales{bits}"], data[f"biases{bits}"],
                      o.BF16, None, 64, bits, y_dtype=o.F32, threads=1)
        ref = data[f"y{bits}"]
        assert (np.abs(y - ref).max(axis=1) <= 1e-5 * np.abs(ref).max(axis=1)).all()


# ---------------------------------------------------------------------------
# silu: the activation in front of the modulation linears
# ---------------------------------------------------------------------------
def _all_finite_16(o, dtype):
    bits = np.arange(1 << 16, dtype=np.uint32).astype(np.uint16)
    f = o._to_f32(bits, dtype)
    return bits[np.isfinite(f)]


@pytest.mark.parametrize("dtype_name", ["bf16", "f16"])
def test_silu_against_torch_cpu_two_operations(oracle, dtype_name):
    """Every finite 16-bit value: the oracle (float64 sigmoid, two roundings)
    against PyTorch's CPU evaluation of the same two operations in the 16-bit
    type, an independent implementation.  Its float32 exponential may round a
    sigmoid the other way on a rare value: at most one ulp then, on well under a
    percent of the values."""
    import torch

    o = oracle
    dtype, tdt = (o.BF16, torch.bfloat16) if dtype_name == "bf16" else (o.F16, torch.float16)
    bits = _all_finite_16(o, dtype)
    got = o.silu_bits(bits, dtype)
    x = torch.from_numpy(bits.view(np.int16)).view(tdt)
    want = (x * torch.sigmoid(x)).view(torch.int16).numpy().view(np.uint16)
    diff = np.abs(got.astype(np.int32) - want.astype(np.int32))
    diff = np.where((got & 0x7FFF) + (want & 0x7FFF) == 0, 0, diff)  # +0 and -0
    assert diff.max() <= 1
    assert (diff != 0).mean() < 0.01


def test_silu_closed_forms(oracle):
    o = oracle
    f = lambda v: float(o.bf16_bits_to_f32(o.silu_bits(o.f32_to_bf16_bits(np.float32([v])), o.BF16))[0])
    assert f(0.0) == 0.0
    assert f(1.0) == 0.73046875          # sigmoid(1) = 0.731058..., bfloat16 0.73046875; times 1
    assert f(64.0) == 64.0 and f(-100.0) == 0.0  # sigmoid saturates: 1, and 0 where the float32 exponential overflows
    assert f(-64.0) == -64.0 * 1.5859375 * 2.0 ** -93   # sigmoid(-64) = e^-64 = 1.58834 * 2^-93 -> 203/128 * 2^-93
    # two roundings, not one: somewhere among all values a single rounding of x * sigmoid(x) must differ
    bits = _all_finite_16(o, o.BF16)
    x = o.bf16_bits_to_f32(bits).astype(np.float64)
    with np.errstate(over="ignore"):
        once = o.f32_to_bf16_bits((x / (1.0 + np.exp(-x))).astype(np.float32))
    assert (once != o.silu_bits(bits, o.BF16)).any(), "the oracle must round the sigmoid before the product"


def test_silu_shape_properties(oracle):
    o = oracle
    bits = _all_finite_16(o, o.BF16)
    x = o.bf16_bits_to_f32(bits)
    y = o.bf16_bits_to_f32(o.silu_bits(bits, o.BF16))
    assert np.all(y[x >= 0] >= 0) and np.all(y[x >= 0] <= x[x >= 0])
    assert np.all(y[x < 0] <= 0) and np.all(y >= np.float32(-0.28))     # minimum of silu is -0.2785
    big = x > 20
    assert np.array_equal(y[big], x[big])
    order = np.argsort(x[x >= 0])
    assert np.all(np.diff(y[x >= 0][order]) >= 0)                          # monotone on the positive side


def test_oracle_clean_under_host_sanitizers():
    """`make -C oracle sanitize`: the C restatement under AddressSanitizer and
    UndefinedBehaviorSanitizer on exactly-sized buffers, every entry point, all
    storage types, bit widths and group sizes."""
    import os
    import subprocess

    here = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle")
    res = subprocess.run(["make", "-C", here, "-B", "sanitize"], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stdout[-2000:] + res.stderr[-2000:]
    assert "combinations clean" in res.stdout
