"""GPU parity: libmfq's quantize / dequantize against the CPU oracle,
bit for bit, through the C ABI (ctypes)."""
import numpy as np
import pytest
import torch

from cases import adversarial_groups as _adversarial_groups, seeded, storage as _storage

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("gs", [32, 64, 128])
@pytest.mark.parametrize("dtype_name", ["bf16", "f16", "f32"])
def test_quantize_bit_exact_random_and_adversarial(oracle, bits, gs, dtype_name):
    import mflux_amd
    from gpu_util import raw, to_dev

    o = oracle
    dtype = {"bf16": o.BF16, "f16": o.F16, "f32": o.F32}[dtype_name]
    rows, K = 96, 1024
    rnd = seeded(9, bits * 1000 + gs, (rows, K), 0.02)
    adv = _adversarial_groups(o, rows * K // gs, gs, seed=bits + gs).reshape(rows, K)
    for name, f32 in (("random", rnd), ("adversarial", adv)):
        w = _storage(o, f32, dtype)
        exp = o.c_quantize(w, dtype, gs, bits)
        got = mflux_amd.quantize(to_dev(w, dtype), group_size=gs, bits=bits)
        torch.cuda.synchronize()
        for what, e, g in zip(("wq", "scales", "biases"), exp, got):
            assert tuple(g.shape) == e.shape, (name, what)
            ge = raw(g)
            bad = np.flatnonzero(ge.reshape(-1) != e.reshape(-1))
            assert bad.size == 0, f"{name}/{what}: {bad.size} mismatches, first at {bad[:4]}"


@pytest.mark.parametrize("bits,N,K", [(4, 3072, 3072), (8, 2048, 3072), (4, 1024, 15360)])
def test_quantize_bit_exact_model_shapes(oracle, bits, N, K):
    import mflux_amd
    from gpu_util import raw, to_dev

    o = oracle
    w = o.f32_to_bf16_bits(seeded(3, bits, (N, K), 0.02))
    exp = o.c_quantize(w, o.BF16, 64, bits)
    got = mflux_amd.quantize(to_dev(w, o.BF16), group_size=64, bits=bits)
    for e, g in zip(exp, got):
        assert np.array_equal(raw(g), e)


def test_quantize_leading_dims_and_tail(oracle):
    """3-D input and a chunk count that does not fill the last wavefront."""
    import mflux_amd
    from gpu_util import raw, to_dev

    o = oracle
    w = o.f32_to_bf16_bits(seeded(9, 77, (3, 5, 96), 1.0))
    exp = o.c_quantize(w, o.BF16, 32, 4)
    got = mflux_amd.quantize(to_dev(w, o.BF16), group_size=32, bits=4)
    for e, g in zip(exp, got):
        assert tuple(g.shape) == e.shape
        assert np.array_equal(raw(g), e)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("gs", [32, 64, 128])
def test_dequantize_two_roundings(oracle, bits, gs):
    """dequantize is bit for bit the oracle's mlxo_dequantize: mx.dequantize is an
    element-wise multiply and an element-wise add on arrays of the scales' type,
    so the product is rounded to bfloat16 before the bias is added and the sum is
    rounded again.  float32 output from bfloat16 scales: code * scale has at most
    16 significant bits, so the two float32 operations equal the exact value
    rounded once."""
    import mflux_amd
    from gpu_util import raw, to_dev, u32_to_dev

    o = oracle
    w = o.f32_to_bf16_bits(seeded(9, 5, (64, 1024), 0.02))
    wq, s, b = o.c_quantize(w, o.BF16, gs, bits)
    exp_bf16 = o.c_dequantize(wq, s, b, o.BF16, gs, bits)
    once = o.f32_to_bf16_bits(o.dequantize_exact(wq, s, b, o.BF16, gs, bits).astype(np.float32))
    assert (exp_bf16 != once).any(), "the case must tell one rounding from two"
    d = mflux_amd.dequantize(u32_to_dev(wq), to_dev(s, o.BF16), to_dev(b, o.BF16), group_size=gs, bits=bits)
    assert d.dtype == torch.bfloat16
    assert np.array_equal(raw(d), exp_bf16)
    d32 = mflux_amd.dequantize(u32_to_dev(wq), to_dev(s, o.BF16), to_dev(b, o.BF16), group_size=gs, bits=bits,
                               dtype=torch.float32)
    assert np.array_equal(raw(d32), o.c_dequantize(wq, s, b, o.BF16, gs, bits, out_dtype=o.F32))
    assert np.array_equal(raw(d32), o.dequantize_exact(wq, s, b, o.BF16, gs, bits).astype(np.float32))


def test_quantize_dequantize_error_bound_full_size():
    """At the full single-block shape: every group reproduces its edge element
    exactly (bias is the edge, code 0); the error of every other element is at
    most one step (re-fitting the scale to the edge can shrink it by up to
    1/16, which clips the far end by up to one code) and typically half a
    step."""
    import mflux_amd

    torch.manual_seed(3001)
    w = (torch.randn(21504, 3072, device="cuda") * 0.02).to(torch.bfloat16)
    wq, s, b = mflux_amd.quantize(w, 64, 4)
    d = mflux_amd.dequantize(wq, s, b, 64, 4, dtype=torch.float32)
    err = (d - w.float()).abs().reshape(21504, 48, 64)
    step = s.float().abs().reshape(21504, 48, 1)
    assert bool((err <= step * (1.0 + 15 * 2.0 ** -9) + 1e-12).all())
    assert float((err <= step * (0.5 + 15 * 2.0 ** -9)).float().mean()) > 0.99
    assert bool((err.amin(dim=2) == 0).all())


@pytest.mark.parametrize("bits", [4, 8])
def test_quantize_bit_exact_wide_exponent_sweep(oracle, bits):
    """2^25 float32 elements whose groups sweep the exponent range (including
    the ranges where the kernel switches between its shared-reciprocal division
    and the compiler's full division) and whose values land on and next to code
    boundaries: every packed word, scale and bias must equal the oracle's."""
    import mflux_amd
    from gpu_util import raw, to_dev

    o = oracle
    rng = np.random.default_rng(77 + bits)
    n_groups, gs = 1 << 19, 64
    n_bins = (1 << bits) - 1
    expo = rng.integers(-80, 60, size=(n_groups, 1)).astype(np.float32)
    base = rng.standard_normal((n_groups, gs), dtype=np.float32)
    # a third of the groups: values placed on exact half-code positions of a power-of-two grid
    grid = (rng.integers(0, 2 * n_bins + 1, size=(n_groups, gs)).astype(np.float32) * np.float32(0.5)
            - np.float32(n_bins // 2))
    kind = rng.integers(0, 3, size=(n_groups, 1))
    f = np.where(kind == 0, grid, base) * np.exp2(expo)
    # another third keeps full float32 mantissas; nudge some values by one ulp
    nudge = rng.integers(-1, 2, size=f.shape).astype(np.int32)
    f = (f.view(np.int32) + np.where(kind == 2, nudge, 0)).view(np.float32)
    f = np.where(np.isfinite(f), f, np.float32(0)).astype(np.float32).reshape(1 << 12, -1)
    exp = o.c_quantize(f, o.F32, gs, bits)
    got = mflux_amd.quantize(to_dev(f, o.F32), group_size=gs, bits=bits)
    for what, e, g in zip(("wq", "scales", "biases"), exp, got):
        bad = np.flatnonzero(raw(g).reshape(-1) != e.reshape(-1))
        assert bad.size == 0, f"{what}: {bad.size} mismatches, first at {bad[:4]}"


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("gs", [32, 64, 128])
def test_dequantize_rows_is_gather_then_dequantize(oracle, bits, gs):
    """The embedding lookup equals dequantize() of the gathered rows, bit for
    bit, for repeated, negative and out-of-range indices and any index shape."""
    import mflux_amd
    from gpu_util import raw, to_dev, u32_to_dev

    o = oracle
    rows, K = 300, 1024
    w = o.f32_to_bf16_bits(seeded(9, 60 + bits, (rows, K), 0.05))
    wq, s, b = o.c_quantize(w, o.BF16, gs, bits)
    full = o.c_dequantize(wq, s, b, o.BF16, gs, bits)  # product and sum each rounded, as mx.dequantize does
    idx = np.array([[0, 299, 7, 7], [-1, -300, 150, 3], [1000, -1000, 42, 299]], dtype=np.int64)
    expect_rows = np.array([[0, 299, 7, 7], [299, 0, 150, 3], [299, 0, 42, 299]])
    args = (u32_to_dev(wq), to_dev(s, o.BF16), to_dev(b, o.BF16))
    got = mflux_amd.dequantize_rows(*args, torch.from_numpy(idx).cuda(), group_size=gs, bits=bits)
    assert tuple(got.shape) == (3, 4, K) and got.dtype == torch.bfloat16
    assert np.array_equal(raw(got), full[expect_rows])
    got32 = mflux_amd.dequantize_rows(*args, torch.tensor([5, 6], dtype=torch.int32).cuda(), group_size=gs, bits=bits,
                                      dtype=torch.float32)
    assert np.array_equal(raw(got32), o.dequantize_exact(wq, s, b, o.BF16, gs, bits).astype(np.float32)[[5, 6]])
    empty = mflux_amd.dequantize_rows(*args, torch.zeros((0,), dtype=torch.int64).cuda(), group_size=gs, bits=bits)
    assert tuple(empty.shape) == (0, K)


def test_quantized_embedding_module(oracle):
    """nn.quantize with the default predicate turns an Embedding into a
    QuantizedEmbedding whose lookup and as_linear agree with the oracle."""
    import mflux_amd
    from gpu_util import raw
    from mflux_amd import nn as qnn

    o = oracle
    torch.manual_seed(5)
    model = torch.nn.Sequential(qnn.Embedding(500, 256)).to(device="cuda", dtype=torch.bfloat16)
    table = raw(model[0].weight)
    qnn.quantize(model, bits=8)
    q = model[0]
    assert isinstance(q, qnn.QuantizedEmbedding) and (q.bits, q.group_size, q.num_embeddings, q.dims) == (8, 64, 500, 256)
    wq, s, b = o.c_quantize(table, o.BF16, 64, 8)
    assert np.array_equal(raw(q.weight), wq) and np.array_equal(raw(q.scales), s) and np.array_equal(raw(q.biases), b)
    ids = torch.tensor([[1, 2, 3], [499, 0, 2]], device="cuda")
    full = o.c_dequantize(wq, s, b, o.BF16, 64, 8)
    assert np.array_equal(raw(model(ids)), full[ids.cpu().numpy()])
    x = torch.randn(3, 256, device="cuda").to(torch.bfloat16)
    y = q.as_linear(x)
    ref = o.quantized_matmul_f64(x.double().cpu().numpy(), wq, s, b, o.BF16, 64, 8)
    err = np.abs(y.double().cpu().numpy() - ref).max(axis=1) / np.abs(ref).max(axis=1)
    assert tuple(y.shape) == (3, 500) and err.max() <= 1e-2


@pytest.mark.parametrize("bits", [3, 5, 6])
@pytest.mark.parametrize("gs", [32, 64, 128])
@pytest.mark.parametrize("dtype_name", ["bf16", "f16"])
def test_odd_bit_widths_quantize_and_dequantize_bit_exact(oracle, bits, gs, dtype_name):
    """3-, 5- and 6-bit packing (MLX's byte packs): packed words, scales and
    biases equal the oracle's; dequantize and the row lookup equal the
    single-rounded fma of the oracle's codes."""
    import mflux_amd
    from gpu_util import TORCH_DT, raw, to_dev, u32_to_dev

    o = oracle
    dtype = {"bf16": o.BF16, "f16": o.F16}[dtype_name]
    rows, K = 80, 1024
    rnd = seeded(9, bits * 1000 + gs + 7, (rows, K), 0.02)
    adv = _adversarial_groups(o, rows * K // gs, gs, seed=bits + gs + 1).reshape(rows, K)
    for name, f32 in (("random", rnd), ("adversarial", adv)):
        w = _storage(o, f32, dtype)
        exp = o.c_quantize(w, dtype, gs, bits)
        got = mflux_amd.quantize(to_dev(w, dtype), group_size=gs, bits=bits)
        for what, e, g in zip(("wq", "scales", "biases"), exp, got):
            assert tuple(g.shape) == e.shape, (name, what)
            bad = np.flatnonzero(raw(g).reshape(-1) != e.reshape(-1))
            assert bad.size == 0, f"{name}/{what}: {bad.size} mismatches, first at {bad[:4]}"
    wq, s, b = exp
    finite = np.isfinite(o.dequantize_exact(wq, s, b, dtype, gs, bits)).all(axis=1)
    with np.errstate(all="ignore"):
        fma32 = o.dequantize_exact(wq, s, b, dtype, gs, bits).astype(np.float32)
    d32 = mflux_amd.dequantize(u32_to_dev(wq), to_dev(s, dtype), to_dev(b, dtype), group_size=gs, bits=bits,
                               dtype=torch.float32)
    assert np.array_equal(raw(d32)[finite], fma32[finite])
    d16 = mflux_amd.dequantize(u32_to_dev(wq), to_dev(s, dtype), to_dev(b, dtype), group_size=gs, bits=bits)
    assert d16.dtype == TORCH_DT[dtype]
    with np.errstate(all="ignore"):
        exp16 = o.c_dequantize(wq, s, b, dtype, gs, bits)  # product and sum each rounded to the type
    ok = finite[:, None] & ~np.isnan(o._to_f32(exp16, dtype))  # a NaN's sign and payload are the machine's choice
    assert np.array_equal(raw(d16)[ok], exp16[ok])
    idx = torch.tensor([[3, -1], [0, 500]], device="cuda")
    looked = mflux_amd.dequantize_rows(u32_to_dev(wq), to_dev(s, dtype), to_dev(b, dtype), idx, group_size=gs,
                                       bits=bits, dtype=torch.float32)
    assert torch.equal(looked, d32[torch.tensor([[3, rows - 1], [0, rows - 1]], device="cuda")])


def test_odd_bit_widths_full_size_weight(oracle):
    """The 5-bit pack over a full FLUX attention weight."""
    import mflux_amd
    from gpu_util import raw, to_dev

    o = oracle
    w = o.f32_to_bf16_bits(seeded(3, 55, (3072, 3072), 0.02))
    exp = o.c_quantize(w, o.BF16, 64, 5)
    got = mflux_amd.quantize(to_dev(w, o.BF16), group_size=64, bits=5)
    for e, g in zip(exp, got):
        assert np.array_equal(raw(g), e)


@pytest.mark.parametrize("bits", [3, 5, 6])
@pytest.mark.parametrize("gs", [32, 64, 128])
def test_odd_bit_widths_float32_input_bit_exact(oracle, bits, gs):
    """float32 weights at 3, 5 and 6 bits: packed words and the float32 scales and
    biases equal the oracle's on random, adversarial (ties, equal groups, tiny and
    huge ranges, denormals) and exponent-sweeping groups; dequantize returns
    the float32 product and sum of the same codes."""
    import mflux_amd
    from gpu_util import raw, to_dev, u32_to_dev

    o = oracle
    rows, K = 96, 1024
    rng = np.random.default_rng(500 + 10 * bits + gs)
    rnd = seeded(9, bits * 1000 + gs + 11, (rows, K), 0.02)
    adv = _adversarial_groups(o, rows * K // gs, gs, seed=bits + gs + 3).reshape(rows, K)
    sweep = (rng.standard_normal((rows * K // gs, gs), dtype=np.float32)
             * np.exp2(rng.integers(-80, 60, size=(rows * K // gs, 1)).astype(np.float32))).reshape(rows, K)
    for name, f32 in (("random", rnd), ("adversarial", adv), ("sweep", sweep)):
        f32 = np.ascontiguousarray(f32, dtype=np.float32)
        exp = o.c_quantize(f32, o.F32, gs, bits)
        got = mflux_amd.quantize(to_dev(f32, o.F32), group_size=gs, bits=bits)
        for what, e, g in zip(("wq", "scales", "biases"), exp, got):
            assert tuple(g.shape) == e.shape, (name, what)
            bad = np.flatnonzero(raw(g).reshape(-1) != e.reshape(-1))
            assert bad.size == 0, f"{name}/{what}: {bad.size} mismatches, first at {bad[:4]}"
        assert got[1].dtype == torch.float32 and got[2].dtype == torch.float32
    wq, s, b = exp
    with np.errstate(all="ignore"):
        exp32 = o.c_dequantize(wq, s, b, o.F32, gs, bits)
    d32 = mflux_amd.dequantize(u32_to_dev(wq), to_dev(s, o.F32), to_dev(b, o.F32), group_size=gs, bits=bits)
    ok = np.isfinite(exp32)
    assert d32.dtype == torch.float32 and np.array_equal(raw(d32)[ok], exp32[ok])
