"""GPU parity: libmfq's quantized matmul (GEMV for M <= 16, MFMA GEMM above)
against the float64 matmul oracle on MLX-format operands.

Tolerance of this path: max |y - y_ref| <= 1e-2 * max|y_ref row|,
per output row.
"""
import numpy as np
import pytest
import torch

from conftest import seeded

pytestmark = pytest.mark.gpu

TOL = 1e-2


def _case(o, cfg, M, K, N, bits, gs=64, with_bias=True, x_std=1.0):
    x = o.f32_to_bf16_bits(seeded(cfg, 0, (M, K), x_std))
    w = o.f32_to_bf16_bits(seeded(cfg, 1, (N, K), 0.02))
    bias = o.f32_to_bf16_bits(seeded(cfg, 2, (N,), 0.02)) if with_bias else None
    wq, s, b = o.c_quantize(w, o.BF16, gs, bits)
    return x, wq, s, b, bias


def _run(o, x, wq, s, b, bias, bits, gs=64):
    import mflux_amd
    from gpu_util import to_dev, u32_to_dev

    y = mflux_amd.quantized_matmul(
        to_dev(x, o.BF16), u32_to_dev(wq), to_dev(s, o.BF16), to_dev(b, o.BF16),
        transpose=True, group_size=gs, bits=bits, bias=None if bias is None else to_dev(bias, o.BF16))
    torch.cuda.synchronize()
    return y


def _ref(o, x, wq, s, b, bias, bits, gs=64):
    xf = o.bf16_bits_to_f32(x).astype(np.float64)
    bf = None if bias is None else o.bf16_bits_to_f32(bias).astype(np.float64)
    return o.quantized_matmul_f64(xf, wq, s, b, o.BF16, gs, bits, bias_f64=bf)


def _assert_close(y: torch.Tensor, ref: np.ndarray, tol=TOL, row_floor=None):
    got = y.detach().to(torch.float64).cpu().numpy()
    assert got.shape == ref.shape
    row_inf = np.abs(ref).max(axis=-1, keepdims=True)
    if row_floor is not None:
        row_inf = np.maximum(row_inf, row_floor)
    err = np.abs(got - ref) / np.maximum(row_inf, 1e-30)
    worst = float(err.max())
    assert worst <= tol, f"max |err| / ||row||inf = {worst:.4g} > {tol}"
    return worst


# ---- GEMV path (M <= 16) ----------------------------------------------------
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("M", [1, 2, 4, 7, 16])
def test_qmv_vs_f64(oracle, bits, M):
    o = oracle
    args = _case(o, 2, M, 3072, 2048 + 16, bits)
    _assert_close(_run(o, *args, bits), _ref(o, *args, bits))


@pytest.mark.parametrize("bits,gs,K,N", [(4, 32, 96, 40), (8, 32, 32, 7), (4, 128, 640, 33), (8, 128, 384, 64),
                                         (4, 64, 64, 16), (8, 64, 192, 1)])
def test_qmv_ragged_shapes(oracle, bits, gs, K, N):
    o = oracle
    args = _case(o, 21, 3, K, N, bits, gs=gs)
    _assert_close(_run(o, *args, bits, gs), _ref(o, *args, bits, gs))


@pytest.mark.parametrize("bits,gs,K", [
    (8, 64, 256), (8, 64, 768), (8, 64, 1024), (8, 64, 1088), (8, 64, 3840), (8, 64, 4096), (8, 64, 5120),
    (8, 64, 6144), (8, 64, 6208),              # 1..6 loads per row, whole and partial last load; 6208: 7 loads
    (4, 64, 3072), (4, 64, 3840), (4, 64, 8192), (4, 64, 12288), (4, 64, 15360),
    (8, 32, 3072), (4, 32, 1024), (4, 32, 96),  # more than 64 groups / odd group count: per-lane scale loads
    (8, 128, 3072), (4, 128, 2048), (8, 128, 384),
])
def test_qmv_single_row_kernel_shapes(oracle, bits, gs, K):
    """M = 1 over every number of loads per row the one-row kernel is built
    for, both ways of fetching scales, and the first shape beyond it."""
    o = oracle
    N = 203  # not a multiple of the wavefront count: uneven runs of rows
    args = _case(o, 22, 1, K, N, bits, gs=gs)
    _assert_close(_run(o, *args, bits, gs), _ref(o, *args, bits, gs))


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("M", [2, 3, 4])
def test_qmv_few_rows_short_k(oracle, bits, M):
    """M = 2..4 with rows of one load: the four-row instantiation, including
    its zero rows (M = 2, 3) and fewer features than wavefronts."""
    o = oracle
    for K, N in ((256, 3072), (768, 50), (1024 if bits == 8 else 2048, 3)):
        args = _case(o, 23, M, K, N, bits)
        _assert_close(_run(o, *args, bits), _ref(o, *args, bits))


@pytest.mark.parametrize("bits,gs,K", [
    (8, 64, 256), (8, 64, 512), (8, 64, 768), (8, 64, 1024), (8, 64, 1536), (8, 64, 2048), (8, 64, 3072), (8, 64, 4096),
    (4, 64, 512), (4, 64, 1024), (4, 64, 1536), (4, 64, 2048), (4, 64, 3072), (4, 64, 4096),
    (8, 128, 3072), (4, 128, 4096), (8, 32, 1024), (4, 32, 2048), (8, 32, 256),
])
@pytest.mark.parametrize("M", [2, 4])
def test_qmv_four_rows_at_a_time(oracle, bits, gs, K, M):
    """M = 2..4 through the kernel that takes four weight rows at a time: every
    number of 256-byte pieces per row it is built for, all group sizes, runs of
    quads of uneven length, bf16 with bias and float32 output."""
    import mflux_amd
    from gpu_util import to_dev, u32_to_dev

    o = oracle
    N = 4 * 1031 if K <= 1024 else 4 * 53
    args = _case(o, 41, M, K, N, bits, gs=gs)
    ref = _ref(o, *args, bits, gs)
    _assert_close(_run(o, *args, bits, gs), ref)
    x, wq, s, b, bias = args
    y32 = mflux_amd.quantized_matmul(to_dev(x, o.BF16).float(), u32_to_dev(wq), to_dev(s, o.BF16), to_dev(b, o.BF16),
                                     group_size=gs, bits=bits, bias=to_dev(bias, o.BF16))
    assert y32.dtype == torch.float32
    _assert_close(y32, ref, tol=2e-3)  # nothing is rounded to 16 bits on this path


def test_qmv_four_rows_one_hot(oracle):
    """One-hot activation rows (a different k in each of the four rows) return
    four columns of the weight: every (piece, block, word) position of the
    four-rows-at-a-time kernel against scale * code + bias."""
    import mflux_amd
    from gpu_util import to_dev, u32_to_dev

    o = oracle
    K, N = 3072, 64
    w = o.f32_to_bf16_bits(seeded(42, 1, (N, K), 0.02))
    for bits in (4, 8):
        wq, s, b = o.c_quantize(w, o.BF16, 64, bits)
        exact = o.dequantize_exact(wq, s, b, o.BF16, 64, bits).astype(np.float64)
        step = np.abs(o.bf16_bits_to_f32(s).astype(np.float64))
        for k0 in (0, 5, 16, 33, 255, 256, 1000, 2047, 3068):
            ks = [k0, (k0 + 1) % K, (k0 + 17) % K, (k0 + 1531) % K]
            xf = np.zeros((4, K), dtype=np.float32)
            for m, k in enumerate(ks):
                xf[m, k] = 1.0
            y = mflux_amd.quantized_matmul(to_dev(o.f32_to_bf16_bits(xf), o.BF16).float(), u32_to_dev(wq),
                                           to_dev(s, o.BF16), to_dev(b, o.BF16), group_size=64, bits=bits)
            got = y.cpu().numpy().astype(np.float64)
            for m, k in enumerate(ks):
                assert np.all(np.abs(got[m] - exact[:, k]) <= 1e-3 * step[:, k // 64]), (bits, k0, m)


def test_qmv_one_hot_and_float32_output(oracle):
    """One-hot x through the one-row kernel returns a column of the weight, for
    every lane position of every load.  The kernel multiplies x with the raw
    codes and applies scale and bias to the float32 sums, so with float32
    output the column comes back unrounded: within a thousandth of a code step
    of scale * code + bias, and within half a 16-bit unit of the dequantised
    (rounded) weight."""
    import mflux_amd
    from gpu_util import to_dev, u32_to_dev

    o = oracle
    K, N = 3072, 96
    w = o.f32_to_bf16_bits(seeded(24, 1, (N, K), 0.02))
    for bits in (4, 8):
        wq, s, b = o.c_quantize(w, o.BF16, 64, bits)
        exact = o.dequantize_exact(wq, s, b, o.BF16, 64, bits).astype(np.float64)
        deq = o.bf16_bits_to_f32(o.f32_to_bf16_bits(exact.astype(np.float32))).astype(np.float64)
        step = np.abs(o.bf16_bits_to_f32(s).astype(np.float64))
        for k in (0, 1, 7, 8, 15, 16, 31, 32, 63, 64, 1023, 1024, 2047, 2048, 3071):
            xf = np.zeros((1, K), dtype=np.float32)
            xf[0, k] = 1.0
            y = mflux_amd.quantized_matmul(to_dev(o.f32_to_bf16_bits(xf), o.BF16).float(), u32_to_dev(wq),
                                           to_dev(s, o.BF16), to_dev(b, o.BF16), group_size=64, bits=bits)
            assert y.dtype == torch.float32
            got = y.cpu().numpy()[0].astype(np.float64)
            assert np.all(np.abs(got - exact[:, k]) <= 1e-3 * step[:, k // 64]), (bits, k)
            assert np.all(np.abs(got - deq[:, k]) <= 2.0 ** -8 * np.abs(deq[:, k]) + 1e-3 * step[:, k // 64]), (bits, k)


def _one_row_ref(o, x_bits, wq, s, b, bits, gs=64):
    xf = o.bf16_bits_to_f32(x_bits).astype(np.float64)
    return o.quantized_matmul_f64(xf, wq, s, b, o.BF16, gs, bits)


@pytest.mark.parametrize("bits", [4, 8])
def test_qmv_one_row_fixed_point_image_of_x(oracle, bits):
    """The one-row kernel turns x into 15-bit fixed point with one power-of-two
    scale per row.  Small integers stay exact (float32 output reproduces the
    integer result bit for bit); a row whose elements span many orders of
    magnitude loses at most 2^-15 of its largest element per element; tiny and
    huge rows are rescaled without under- or overflow; a zero row gives the
    bias; an infinity in x makes every output NaN."""
    import mflux_amd
    from gpu_util import to_dev, u32_to_dev

    o = oracle
    rng = np.random.default_rng(31 + bits)
    K, N = 3072, 520
    n_bins = 2 ** bits - 1
    codes = rng.integers(0, n_bins + 1, (N, K)).astype(np.float32)
    codes[:, ::64] = 0
    codes[:, 1::64] = n_bins          # every group spans 0..n_bins: scale 1 (or -1), dequantised weight = code
    w_bits = o.f32_to_bf16_bits(codes)
    wq, s, b = o.c_quantize(w_bits, o.BF16, 64, bits)
    assert np.array_equal(o.dequantize_exact(wq, s, b, o.BF16, 64, bits), codes)
    dev = lambda a: to_dev(a, o.BF16)
    run = lambda xb, **kw: mflux_amd.quantized_matmul(dev(xb).float(), u32_to_dev(wq), dev(s), dev(b), group_size=64,
                                                      bits=bits, **kw).cpu().numpy().astype(np.float64)
    # small integers: exact
    xi = rng.integers(-3, 4, (1, K)).astype(np.float32)
    assert np.array_equal(run(o.f32_to_bf16_bits(xi)), xi.astype(np.float64) @ codes.astype(np.float64).T)
    # a wide dynamic range: bound from the rounding of x alone, plus float32 rounding of the sums
    xw = (rng.standard_normal((1, K)) * 10.0 ** rng.integers(-6, 3, (1, K))).astype(np.float32)
    xb = o.f32_to_bf16_bits(xw)
    xmax = np.abs(o.bf16_bits_to_f32(xb)).max()
    ref = _one_row_ref(o, xb, wq, s, b, bits)
    bound = 2.0 ** -15 * xmax * np.abs(codes).sum(axis=1) + 2.0 ** -20 * np.abs(ref)
    assert np.all(np.abs(run(xb) - ref) <= bound)
    # tiny and huge rows (the scale's exponent is clamped for the former), against float64
    for mag in (1e-30, 1e-12, 1e20, 1e30):
        xb = o.f32_to_bf16_bits((rng.standard_normal((1, K)) * mag).astype(np.float32))
        ref = _one_row_ref(o, xb, wq, s, b, bits)
        got = run(xb)
        assert np.all(np.isfinite(got)) and np.all(np.abs(got - ref) <= 1e-3 * np.abs(ref).max())
    # zeros give the bias exactly; an infinity anywhere gives NaN everywhere
    bias = o.f32_to_bf16_bits(seeded(32, 2, (N,), 1.0))
    zero = np.zeros((1, K), dtype=np.uint16)
    assert np.array_equal(run(zero, bias=dev(bias))[0], o.bf16_bits_to_f32(bias).astype(np.float64))
    xinf = o.f32_to_bf16_bits(xi.copy())
    xinf[0, 1000] = 0x7f80
    assert np.all(np.isnan(run(xinf)))


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("M", [2, 3, 4])
def test_qmv_four_rows_fixed_point_images_of_x(oracle, bits, M):
    """The four-rows kernel gives every activation row its own power-of-two
    scale.  Small integers stay exact whatever the other rows hold; rows of very
    different magnitude do not disturb each other; a zero row gives the bias;
    an infinity makes its own row NaN and leaves the others as they were."""
    import mflux_amd
    from gpu_util import to_dev, u32_to_dev

    o = oracle
    rng = np.random.default_rng(77 + 10 * bits + M)
    K, N = 3072, 256
    n_bins = 2 ** bits - 1
    codes = rng.integers(0, n_bins + 1, (N, K)).astype(np.float32)
    codes[:, ::64] = 0
    codes[:, 1::64] = n_bins          # every group spans 0..n_bins: the dequantised weight is the code
    wq, s, b = o.c_quantize(o.f32_to_bf16_bits(codes), o.BF16, 64, bits)
    assert np.array_equal(o.dequantize_exact(wq, s, b, o.BF16, 64, bits), codes)
    dev = lambda a: to_dev(a, o.BF16)
    run = lambda xb, **kw: mflux_amd.quantized_matmul(dev(xb).float(), u32_to_dev(wq), dev(s), dev(b), group_size=64,
                                                      bits=bits, **kw).cpu().numpy().astype(np.float64)
    c64 = codes.astype(np.float64)
    # small integers in every row, each row at its own magnitude (powers of two keep them exact in bfloat16)
    xi = rng.integers(-3, 4, (M, K)).astype(np.float32) * (2.0 ** np.arange(0, 6 * M, 6, dtype=np.float32))[:, None]
    assert np.array_equal(run(o.f32_to_bf16_bits(xi)), xi.astype(np.float64) @ c64.T)
    # rows 1e-12 ... 1e20 side by side: each within its own bound
    mags = np.array([1e-12, 1.0, 1e20, 1e-3][:M], dtype=np.float64)[:, None]
    xb = o.f32_to_bf16_bits((rng.standard_normal((M, K)) * mags).astype(np.float32))
    xf = o.bf16_bits_to_f32(xb).astype(np.float64)
    ref = xf @ c64.T
    got = run(xb)
    bound = 2.0 ** -15 * np.abs(xf).max(axis=1, keepdims=True) * np.abs(c64).sum(axis=1)[None, :] + 2.0 ** -20 * np.abs(ref)
    assert np.all(np.isfinite(got)) and np.all(np.abs(got - ref) <= bound)
    # a zero row gives the bias exactly, next to rows that are not zero
    bias = o.f32_to_bf16_bits(seeded(78, 2, (N,), 1.0))
    xz = xb.copy()
    xz[0] = 0
    got = run(xz, bias=dev(bias))
    assert np.array_equal(got[0], o.bf16_bits_to_f32(bias).astype(np.float64))
    # an infinity: its row is NaN, the other rows unchanged
    base = run(xb)
    xinf = xb.copy()
    xinf[1, 1000] = 0x7f80
    got = run(xinf)
    assert np.all(np.isnan(got[1]))
    keep = [m for m in range(M) if m != 1]
    assert np.array_equal(got[keep], base[keep])



@pytest.mark.parametrize("N", [1, 2, 3, 5, 63, 262144 + 8])
def test_qmv_one_row_run_lengths(oracle, N):
    """Rows are dealt to wavefronts in runs of up to 64 (a lane keeps one
    result until the run ends): fewer rows than wavefronts in a workgroup, odd
    and even runs, and runs of the full 64 rows."""
    o = oracle
    K = 64
    args = _case(o, 33, 1, K, N, 8, with_bias=True)
    _assert_close(_run(o, *args, 8), _ref(o, *args, 8))


def test_qmv_adaln_config_full(oracle):
    """The adaLN modulation shape: SiLU(temb) [M,3072] against W8 [18432,3072]."""
    o = oracle
    for M in (1, 4):
        temb = seeded(2, 0, (M, 3072), 1.0)
        x = o.f32_to_bf16_bits(temb / (1.0 + np.exp(-temb)))
        w = o.f32_to_bf16_bits(seeded(2, 1, (18432, 3072), 0.02))
        bias = o.f32_to_bf16_bits(seeded(2, 2, (18432,), 0.02))
        wq, s, b = o.c_quantize(w, o.BF16, 64, 8)
        _assert_close(_run(o, x, wq, s, b, bias, 8), _ref(o, x, wq, s, b, bias, 8))


# ---- GEMM path ----------------------------------------------------------------
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("M,K,N", [(256, 512, 256), (512, 3072, 768), (300, 256, 200), (17, 64, 64), (1000, 1024, 520)])
def test_qmm_vs_f64(oracle, bits, M, K, N):
    o = oracle
    args = _case(o, 1, M, K, N, bits)
    _assert_close(_run(o, *args, bits), _ref(o, *args, bits))


@pytest.mark.parametrize("bits,gs", [(4, 64), (8, 64), (4, 32), (8, 128)])
@pytest.mark.parametrize("M,K,N", [(512, 3072, 768), (256, 3072, 520), (300, 1024, 200), (40, 2048, 1024)])
def test_qmm_split_k_shapes(oracle, bits, gs, M, K, N):
    """Few output tiles and a long K: the launcher cuts K into ranges that run
    on different compute units and a second kernel adds the float32 planes.
    Same tolerance; bf16 and float32 output; with bias."""
    import mflux_amd
    from gpu_util import to_dev, u32_to_dev
    from mflux_amd import _lib

    o = oracle
    assert _lib.load().mfq_qmm_t_workspace_bytes(M, K, N, gs, bits) >= 2 * M * N * 4, "this shape should be split"
    args = _case(o, 14, M, K, N, bits, gs=gs)
    ref = _ref(o, *args, bits, gs)
    _assert_close(_run(o, *args, bits, gs), ref)
    x, wq, s, b, bias = args
    y32 = mflux_amd.quantized_matmul(to_dev(x, o.BF16).float(), u32_to_dev(wq), to_dev(s, o.BF16), to_dev(b, o.BF16),
                                     group_size=gs, bits=bits, bias=to_dev(bias, o.BF16))
    assert y32.dtype == torch.float32
    _assert_close(y32, ref, tol=5e-3)  # float32 output: only the weights' 16-bit rounding remains


@pytest.mark.parametrize("bits", [4, 8])
def test_qmm_last_round_cut_along_k(oracle, bits):
    """270 tiles on a 256-CU GPU: the first 256 run whole, the 14 of the last
    round are cut along K into float32 planes that a second kernel adds up
    (ragged M and N, bias).  The bf16 call goes through the two-kernel path (its
    workspace: the 16-bit copy of the weights, then the planes), the call with
    float32 activations and output through the fused kernel's cut."""
    import mflux_amd
    from gpu_util import to_dev, u32_to_dev
    from mflux_amd import _lib

    o = oracle
    M, K, N = 2200, 2048, 7504
    if torch.cuda.get_device_properties(0).multi_processor_count == 256:
        assert _lib.load().mfq_qmm_t_workspace_bytes(M, K, N, 64, bits) == N * K * 2 + 14 * 8 * 256 * 256 * 4
    args = _case(o, 34, M, K, N, bits)
    ref = _ref(o, *args, bits)
    _assert_close(_run(o, *args, bits), ref)
    x, wq, s, b, bias = args
    y32 = mflux_amd.quantized_matmul(to_dev(x, o.BF16).float(), u32_to_dev(wq), to_dev(s, o.BF16), to_dev(b, o.BF16),
                                     group_size=64, bits=bits, bias=to_dev(bias, o.BF16))
    assert y32.dtype == torch.float32
    _assert_close(y32, ref, tol=5e-3)


def test_qmm_split_k_matches_unsplit_through_c_abi(oracle):
    """mfq_qmm_t (no workspace) and mfq_qmm_t_ws (split) on the same operands:
    both within tolerance of the oracle and of each other; a too-small
    workspace silently runs unsplit."""
    from gpu_util import to_dev, u32_to_dev
    from mflux_amd import _lib

    o = oracle
    lib = _lib.load()
    M, K, N, bits = 512, 3072, 512, 4
    x, wq, s, b, bias = _case(o, 15, M, K, N, bits)
    ref = _ref(o, x, wq, s, b, bias, bits)
    xd, wd, sd, bd, biasd = to_dev(x, o.BF16), u32_to_dev(wq), to_dev(s, o.BF16), to_dev(b, o.BF16), to_dev(bias, o.BF16)
    need = lib.mfq_qmm_t_workspace_bytes(M, K, N, 64, bits)
    assert need > 0
    outs = []
    for ws_bytes in (0, 16, need):
        y = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device="cuda")
        rc = lib.mfq_qmm_t_ws(xd.data_ptr(), _lib.BF16, M, K, wd.data_ptr(), sd.data_ptr(), bd.data_ptr(), _lib.BF16,
                              biasd.data_ptr(), N, 64, bits, y.data_ptr(), _lib.BF16,
                              ws.data_ptr() if ws_bytes else None, ws_bytes, None)
        assert rc == 0
        torch.cuda.synchronize()
        _assert_close(y, ref)
        outs.append(y)
    assert torch.equal(outs[0], outs[1])                       # too small: same unsplit kernel
    diff = (outs[0].float() - outs[2].float()).abs().max() / outs[0].float().abs().max()
    assert float(diff) <= 1e-2


@pytest.mark.parametrize("bits", [4, 8])
def test_qmm_k_not_multiple_of_64(oracle, bits):
    """Group size 32 allows K = 96: large M goes through the small-M kernel in
    slices of 16 rows (x slices are 16-byte aligned: 96 * 2 * 16 bytes)."""
    o = oracle
    args = _case(o, 12, 50, 96, 72, bits, gs=32)
    _assert_close(_run(o, *args, bits, 32), _ref(o, *args, bits, 32))


@pytest.mark.parametrize("bits", [3, 5, 6])
@pytest.mark.parametrize("M", [1, 300])
def test_odd_bit_widths_matmul(oracle, bits, M):
    """3, 5, 6 bits, one row (its own kernel) and a few hundred (the
    128-column-tile GEMM on the bit stream), through the functional API and
    through a QuantizedLinear."""
    import mflux_amd
    from gpu_util import to_dev
    from mflux_amd import nn as qnn

    o = oracle
    args = _case(o, 13, M, 512, 192, bits)
    ref = _ref(o, *args, bits)
    _assert_close(_run(o, *args, bits), ref)
    x, wq, s, b, bias = args
    lin = qnn.Linear(512, 192, bias=True, device="cuda", dtype=torch.bfloat16)
    with torch.no_grad():
        lin.weight.copy_(to_dev(o.f32_to_bf16_bits(seeded(13, 1, (192, 512), 0.02)), o.BF16))
        lin.bias.copy_(to_dev(bias, o.BF16))
    q = lin.to_quantized(bits=bits)
    assert q.bits == bits and tuple(q.weight.shape) == (192, 512 * bits // 32)
    _assert_close(q(to_dev(x, o.BF16)), ref)


@pytest.mark.parametrize("bits", [3, 5, 6])
@pytest.mark.parametrize("gs,K", [(64, 3072), (64, 4096), (64, 8192), (64, 2048), (32, 96), (32, 1056), (128, 6144),
                                  (64, 8256)])
def test_odd_bit_widths_single_row_kernel(oracle, bits, gs, K):
    """3, 5, 6 bits with one activation row: the fused kernel (one to four units
    of 32 codes per lane, whole and partial last rounds, all group sizes) and,
    for K = 8256, the first shape beyond it (the GEMM kernel with one row)."""
    import mflux_amd
    from gpu_util import to_dev, u32_to_dev

    o = oracle
    N = 203
    args = _case(o, 51, 1, K, N, bits, gs=gs)
    ref = _ref(o, *args, bits, gs)
    _assert_close(_run(o, *args, bits, gs), ref)
    x, wq, s, b, bias = args
    y32 = mflux_amd.quantized_matmul(to_dev(x, o.BF16).float(), u32_to_dev(wq), to_dev(s, o.BF16), to_dev(b, o.BF16),
                                     group_size=gs, bits=bits, bias=to_dev(bias, o.BF16))
    assert y32.dtype == torch.float32
    _assert_close(y32, ref, tol=5e-3)


@pytest.mark.parametrize("bits", [3, 5, 6])
def test_odd_bit_widths_one_hot(oracle, bits):
    """One-hot x picks single weights out of the bit stream: every code position
    of a unit, units of both rounds, against scale * code + bias."""
    import mflux_amd
    from gpu_util import to_dev, u32_to_dev

    o = oracle
    K, N = 3072, 48
    w = o.f32_to_bf16_bits(seeded(52, 1, (N, K), 0.02))
    wq, s, b = o.c_quantize(w, o.BF16, 64, bits)
    exact = o.dequantize_exact(wq, s, b, o.BF16, 64, bits).astype(np.float64)
    step = np.abs(o.bf16_bits_to_f32(s).astype(np.float64))
    for k in list(range(0, 32)) + [32, 63, 64, 1000, 2047, 2048, 2049, 2079, 3040, 3071]:
        xf = np.zeros((1, K), dtype=np.float32)
        xf[0, k] = 1.0
        y = mflux_amd.quantized_matmul(to_dev(o.f32_to_bf16_bits(xf), o.BF16).float(), u32_to_dev(wq),
                                       to_dev(s, o.BF16), to_dev(b, o.BF16), group_size=64, bits=bits)
        got = y.cpu().numpy()[0].astype(np.float64)
        assert np.all(np.abs(got - exact[:, k]) <= 1e-3 * step[:, k // 64]), (bits, k)


def test_odd_bit_widths_c_abi_coverage(oracle):
    """mfq_qmm_t takes 3-, 5- and 6-bit weights for any number of rows: one row of
    at most 8192 codes on its own kernel, the rest on the GEMM kernel."""
    from gpu_util import to_dev, u32_to_dev
    from mflux_amd import _lib

    o = oracle
    lib = _lib.load()
    for bits in (3, 5, 6):
        for M, K in ((1, 3072), (2, 3072), (1, 8256)):
            args = _case(o, 53, M, K, 16, bits, gs=32, with_bias=False)
            x, wq, s, b, _ = args
            xd, wd, sd, bd = to_dev(x, o.BF16), u32_to_dev(wq), to_dev(s, o.BF16), to_dev(b, o.BF16)
            y = torch.empty((M, 16), dtype=torch.bfloat16, device="cuda")
            rc = lib.mfq_qmm_t(xd.data_ptr(), _lib.BF16, M, K, wd.data_ptr(), sd.data_ptr(), bd.data_ptr(), _lib.BF16,
                               None, 16, 32, bits, y.data_ptr(), _lib.BF16, None)
            torch.cuda.synchronize()
            assert rc == 0, (bits, M, K, rc)
            _assert_close(y, _ref(o, *args, bits, 32))


def test_odd_bit_widths_single_row_f16(oracle):
    import mflux_amd
    from gpu_util import raw

    o = oracle
    torch.manual_seed(5)
    for bits in (3, 5, 6):
        x = torch.randn(1, 3072, device="cuda").to(torch.float16)
        w = (torch.randn(130, 3072, device="cuda") * 0.02).to(torch.float16)
        wq, s, b = mflux_amd.quantize(w, 64, bits)
        y = mflux_amd.quantized_matmul(x, wq, s, b, bits=bits)
        ref = o.quantized_matmul_f64(x.double().cpu().numpy(), raw(wq), raw(s), raw(b), o.F16, 64, bits)
        _assert_close(y, ref)


@pytest.mark.parametrize("bits,gs", [(4, 32), (8, 32), (4, 128), (8, 128)])
def test_qmm_group_sizes(oracle, bits, gs):
    o = oracle
    args = _case(o, 11, 320, 512, 384, bits, gs=gs, with_bias=False)
    _assert_close(_run(o, *args, bits, gs), _ref(o, *args, bits, gs))


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("M", [5, 64])
def test_one_hot_rows_return_dequantised_weight_rows(oracle, bits, M):
    """x = one-hot rows: y[m, :] must be column k_m of the dequantised weight,
    which pins the packing order and the tile layout end to end (exactly: one
    product, no accumulation error beyond the bf16 rounding of the weight)."""
    o = oracle
    K, N = 512, 320
    w = o.f32_to_bf16_bits(seeded(5, 1, (N, K), 0.02))
    wq, s, b = o.c_quantize(w, o.BF16, 64, bits)
    ks = (np.arange(M) * 37 + 3) % K
    xf = np.zeros((M, K), dtype=np.float32)
    xf[np.arange(M), ks] = 1.0
    x = o.f32_to_bf16_bits(xf)
    y = _run(o, x, wq, s, b, None, bits)
    exact = o.dequantize_exact(wq, s, b, o.BF16, 64, bits)  # [N, K]
    exp = o.f32_to_bf16_bits(exact[:, ks].T.astype(np.float32))
    from gpu_util import raw
    assert np.array_equal(raw(y), exp)


@pytest.mark.parametrize("bits", [4, 8])
def test_integer_weights_exact(oracle, bits):
    """scale = 1, bias = 0, small integer x: the product is an integer matmul
    that float32 accumulation represents exactly."""
    import mflux_amd
    from gpu_util import to_dev, u32_to_dev, raw

    o = oracle
    rng = np.random.default_rng(42)
    M, K, N = 272, 128, 96
    codes = rng.integers(0, 1 << bits, (N, K)).astype(np.uint32)
    per = 32 // bits
    wq = np.bitwise_or.reduce(codes.reshape(N, K // per, per) << (np.arange(per, dtype=np.uint32) * bits), axis=2)
    s = o.f32_to_bf16_bits(np.ones((N, K // 64), dtype=np.float32))
    b = o.f32_to_bf16_bits(np.zeros((N, K // 64), dtype=np.float32))
    xi = rng.integers(-2, 3, (M, K)).astype(np.float32)
    y = mflux_amd.quantized_matmul(to_dev(o.f32_to_bf16_bits(xi), o.BF16).float(), u32_to_dev(wq.astype(np.uint32)),
                                   to_dev(s, o.BF16), to_dev(b, o.BF16), group_size=64, bits=bits)
    assert y.dtype == torch.float32
    exp = xi.astype(np.int64) @ codes.astype(np.int64).T
    assert np.array_equal(raw(y).astype(np.int64), exp)


@pytest.mark.parametrize("shape", ["linear1", "linear2"])
def test_qmm_flux_single_block_full_size(oracle, shape):
    """The FLUX.1 single-block linears at full size: sampled rows against the float64 oracle,
    and linearity y(x1 + x2) ~ y(x1) + y(x2) on the whole output."""
    import mflux_amd
    from gpu_util import to_dev, u32_to_dev

    o = oracle
    M = 4608
    K, N = (3072, 21504) if shape == "linear1" else (15360, 3072)
    torch.manual_seed(3000 + (shape == "linear2"))
    x = torch.randn(M, K, device="cuda").to(torch.bfloat16)
    w = (torch.randn(N, K, device="cuda") * 0.02).to(torch.bfloat16)
    wq, s, b = mflux_amd.quantize(w, 64, 4)
    y = mflux_amd.quantized_matmul(x, wq, s, b, group_size=64, bits=4)
    rows = np.array([0, 1, 255, 256, 1234, 2303, 2304, 4095, 4351, 4607])
    from gpu_util import raw
    xs = o.bf16_bits_to_f32(raw(x[rows])).astype(np.float64)
    ref = o.quantized_matmul_f64(xs, raw(wq), raw(s), raw(b), o.BF16, 64, 4)
    _assert_close(y[rows], ref)
    # independent GPU cross-check of every element: dense bf16 matmul on the dequantised weight
    dense = torch.matmul(x, mflux_amd.dequantize(wq, s, b, 64, 4).t()).float()
    row_inf = dense.abs().amax(dim=1, keepdim=True)
    assert float(((y.float() - dense).abs() / row_inf).max()) <= 2 * TOL


def test_qmm_ragged_m_qwen(oracle):
    """Qwen-Image image stream M = 6889 = 83^2 (not a tile multiple)."""
    import mflux_amd
    from gpu_util import raw

    o = oracle
    torch.manual_seed(5000)
    M, K, N = 6889, 3072, 3072
    x = torch.randn(M, K, device="cuda").to(torch.bfloat16)
    w = (torch.randn(N, K, device="cuda") * 0.02).to(torch.bfloat16)
    bias = (torch.randn(N, device="cuda") * 0.02).to(torch.bfloat16)
    wq, s, b = mflux_amd.quantize(w, 64, 4)
    guard = torch.full((M + 8, N), 7.0, device="cuda", dtype=torch.bfloat16)
    y = mflux_amd.quantized_matmul(x, wq, s, b, group_size=64, bits=4, bias=bias)
    rows = np.array([0, 6655, 6656, 6800, 6888])
    xs = o.bf16_bits_to_f32(raw(x[rows])).astype(np.float64)
    ref = o.quantized_matmul_f64(xs, raw(wq), raw(s), raw(b), o.BF16, 64, 4,
                                 bias_f64=o.bf16_bits_to_f32(raw(bias)).astype(np.float64))
    _assert_close(y[rows], ref)
    assert bool((guard == 7.0).all())


def test_leading_batch_dims_and_dtype_promotion():
    import mflux_amd

    torch.manual_seed(1)
    w = (torch.randn(128, 256, device="cuda") * 0.02).to(torch.bfloat16)
    wq, s, b = mflux_amd.quantize(w, 64, 4)
    x = torch.randn(1, 40, 256, device="cuda")
    y32 = mflux_amd.quantized_matmul(x, wq, s, b)
    assert y32.shape == (1, 40, 128) and y32.dtype == torch.float32
    y16 = mflux_amd.quantized_matmul(x.to(torch.bfloat16), wq, s, b)
    assert y16.shape == (1, 40, 128) and y16.dtype == torch.bfloat16
    assert float((y32 - y16.float()).abs().max()) < 0.05


@pytest.mark.parametrize("bits", [4, 8])
def test_f16_path(oracle, bits):
    """float16 activations, scales and biases: one activation row (codes enter
    the matrix core as 1024 + code), a few rows, both tile heights of the
    medium-M kernel (with and without a K split) and the large-M kernel."""
    import mflux_amd
    from gpu_util import raw

    o = oracle
    torch.manual_seed(2)
    for M, K, N in ((1, 3072, 200), (3, 512, 192), (100, 512, 192), (300, 2048, 192), (1100, 512, 4200)):
        x = torch.randn(M, K, device="cuda").to(torch.float16)
        w = (torch.randn(N, K, device="cuda") * 0.02).to(torch.float16)
        wq, s, b = mflux_amd.quantize(w, 64, bits)
        e = o.c_quantize(raw(w), o.F16, 64, bits)
        assert np.array_equal(raw(wq), e[0])
        y = mflux_amd.quantized_matmul(x, wq, s, b, bits=bits)
        ref = o.quantized_matmul_f64(x.double().cpu().numpy(), raw(wq), raw(s), raw(b), o.F16, 64, bits)
        _assert_close(y, ref)


@pytest.mark.parametrize("bits,gs", [(4, 64), (8, 64), (4, 32), (8, 32), (4, 128), (8, 128)])
@pytest.mark.parametrize("M,K,N", [(100, 512, 1000), (128, 3072, 136), (129, 1024, 264), (256, 2048, 520),
                                   (400, 768, 130), (77, 768, 3072)])
def test_qmm_medium_m(oracle, bits, gs, M, K, N):
    """The 128-column-tile kernel: 128-row tiles (M <= 128) and 256-row tiles,
    ragged M and N, K with and without a split, a K that is not a whole number
    of scale periods (768 with groups of 128), all group sizes; bf16 with bias
    and float32 output."""
    import mflux_amd
    from gpu_util import to_dev, u32_to_dev

    o = oracle
    args = _case(o, 31, M, K, N, bits, gs=gs)
    ref = _ref(o, *args, bits, gs)
    _assert_close(_run(o, *args, bits, gs), ref)
    x, wq, s, b, bias = args
    y32 = mflux_amd.quantized_matmul(to_dev(x, o.BF16).float(), u32_to_dev(wq), to_dev(s, o.BF16), to_dev(b, o.BF16),
                                     group_size=gs, bits=bits, bias=to_dev(bias, o.BF16))
    assert y32.dtype == torch.float32
    _assert_close(y32, ref, tol=5e-3)


def test_qmm_medium_m_odd_n(oracle):
    """N not a multiple of 4: element-wise guarded stores."""
    o = oracle
    for M, N in ((90, 131), (300, 77)):
        args = _case(o, 32, M, 512, N, 4)
        _assert_close(_run(o, *args, 4), _ref(o, *args, 4))


@pytest.mark.parametrize("bits,gs", [(4, 64), (8, 128)])
def test_qmm_many_rows_long_k_split(oracle, bits, gs):
    """More than 512 rows, few 256 x 256 tiles and K >= 8192: the large-M
    kernel with every tile cut along K across compute units."""
    from mflux_amd import _lib

    o = oracle
    M, K, N = 600, 8192, 256
    assert _lib.load().mfq_qmm_t_workspace_bytes(M, K, N, gs, bits) >= 2 * M * N * 4
    args = _case(o, 33, M, K, N, bits, gs=gs)
    _assert_close(_run(o, *args, bits, gs), _ref(o, *args, bits, gs))


@pytest.mark.parametrize("bits", [4, 8, 5])
def test_transpose_false_and_input_gradient(oracle, bits):
    """transpose=False is g @ dequantize(w); it is also the gradient of the
    fused forward with respect to x, so a LoRA can be trained on a quantized
    base.  Both against float64 on the exactly dequantized weight."""
    import mflux_amd
    from gpu_util import to_dev, u32_to_dev
    from mflux_amd import nn as qnn

    o = oracle
    M, K, N = 40, 512, 192
    x, wq, s, b, bias = _case(o, 16, M, K, N, bits)
    wd, sd, bd = u32_to_dev(wq), to_dev(s, o.BF16), to_dev(b, o.BF16)
    w_exact = o.dequantize_exact(wq, s, b, o.BF16, 64, bits)                       # [N, K]
    g = o.f32_to_bf16_bits(seeded(16, 5, (M, N), 1.0))
    gx = mflux_amd.quantized_matmul(to_dev(g, o.BF16), wd, sd, bd, transpose=False, group_size=64, bits=bits)
    assert tuple(gx.shape) == (M, K) and gx.dtype == torch.bfloat16
    _assert_close(gx, o.bf16_bits_to_f32(g).astype(np.float64) @ w_exact)
    with pytest.raises(ValueError, match="transpose=false"):
        mflux_amd.quantized_matmul(to_dev(x, o.BF16), wd, sd, bd, transpose=False, group_size=64, bits=bits)

    # autograd through a QuantizedLinear wrapped by a LoRA-style branch
    q = qnn.QuantizedLinear(K, N, bias=True, bits=bits, device="cuda")
    q.weight, q.scales, q.biases, q.bias = wd, sd, bd, to_dev(bias, o.BF16)
    xt = to_dev(x, o.BF16).clone().requires_grad_(True)
    a = (torch.randn(K, 4, device="cuda") * 0.05).to(torch.bfloat16).requires_grad_(True)
    bl = (torch.randn(4, N, device="cuda") * 0.05).to(torch.bfloat16).requires_grad_(True)
    y = q(xt) + (xt @ a) @ bl
    y.backward(to_dev(g, o.BF16))
    gf = o.bf16_bits_to_f32(g).astype(np.float64)
    ref_gx = gf @ w_exact + (gf @ bl.detach().double().cpu().numpy().T) @ a.detach().double().cpu().numpy().T
    _assert_close(xt.grad, ref_gx, tol=2e-2)   # two bf16-rounded terms added in bf16
    assert a.grad is not None and bl.grad is not None and q.weight.grad is None
    # and no autograd graph is built when nothing requires grad
    assert not q(to_dev(x, o.BF16)).requires_grad


def test_calls_replay_in_a_hip_graph(oracle):
    """The kernels take everything from their arguments and the current stream
    (no memsets, no host synchronisation), so a sequence of calls can be
    captured once and replayed: one activation row, the medium-M kernel with
    its K cut (workspace from the capture's allocator) and the large-M kernel,
    replayed with eager work and synchronisations in between, every replay
    equal to the eager results bit for bit."""
    import mflux_amd

    torch.manual_seed(9)
    shapes = ((1, 3072, 1024, 8), (300, 2048, 520, 4), (2200, 512, 2304, 4))
    ops = []
    for M, K, N, bits in shapes:
        x = torch.randn(M, K, device="cuda").to(torch.bfloat16)
        w = (torch.randn(N, K, device="cuda") * 0.02).to(torch.bfloat16)
        ops.append((x, *mflux_amd.quantize(w, 64, bits), bits))
    x4 = torch.randn(4, 3072, device="cuda").to(torch.bfloat16)

    def run():
        outs = [mflux_amd.quantized_matmul(x, wq, s, b, bits=bits) for x, wq, s, b, bits in ops]
        # the matvecs with the activation inside (one row, four rows) and the four-rows kernel as it is
        x1, wq, s, b, bits = ops[0]
        outs.append(mflux_amd.silu_quantized_matmul(x1, wq, s, b, bits=bits))
        outs.append(mflux_amd.silu_quantized_matmul(x4, wq, s, b, bits=bits))
        outs.append(mflux_amd.quantized_matmul(x4, wq, s, b, bits=bits))
        return outs

    eager = run()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = run()
    for i in range(3):
        for o in outs:
            o.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        for o, e in zip(outs, eager):
            assert torch.equal(o, e), i
        # eager work between replays
        again = run()
        torch.cuda.synchronize()
        for a, e in zip(again, eager):
            assert torch.equal(a, e)


def _sweep_cases():
    """Seeded shapes that sit on and around the borders between the kernels: the
    row counts where the matvec kernels hand over to each other and to the GEMMs,
    ragged N (odd, below one tile, just past a tile) and K from one group up."""
    rng = np.random.default_rng(20240611)
    m_pool = [1, 2, 3, 4, 5, 8, 15, 16, 17, 31, 33, 63, 64, 65, 127, 128, 129, 130, 255, 257, 511, 513, 700, 1025]
    cases = []
    for i in range(56):
        gs = int(rng.choice([32, 64, 128]))
        bits = int(rng.choice([4, 8, 4, 8, 3, 5, 6]))
        M = int(rng.choice(m_pool))
        if bits in (3, 5, 6) and M > 64:
            M = int(rng.choice([1, 1, 2, 40]))
        K = gs * int(rng.integers(1, 2560 // gs + 1))
        N = int(rng.choice([1, 3, 8, 17, 64, 100, 127, 128, 129, 255, 256, 264, 391, 520, 641]))
        cases.append((i, M, K, N, bits, gs))
    return cases


@pytest.mark.parametrize("case", _sweep_cases(), ids=lambda c: "case%d-M%d-K%d-N%d-w%d-g%d" % c)
def test_shape_sweep_against_oracle(oracle, case):
    o = oracle
    i, M, K, N, bits, gs = case
    args = _case(o, 400 + i, M, K, N, bits, gs=gs, with_bias=bool(i % 2))
    # The bound is relative to a row's largest output.  With one or three output
    # features that largest output can itself be next to nothing (a chance
    # cancellation), so it is held at the size an output of this row has on
    # average, |x row|_2 times the weights' standard deviation.
    x_norm = np.linalg.norm(o.bf16_bits_to_f32(args[0]).astype(np.float64), axis=-1, keepdims=True)
    _assert_close(_run(o, *args, bits, gs), _ref(o, *args, bits, gs), row_floor=0.02 * x_norm)


# The borders that the row count and the tile count draw between the large-M paths: 1024 rows (3, 5 and 6 bits
# move from the 128-column-tile kernel to the two-kernel path; the untransposed product likewise at 4 and 8 bits),
# 2048 rows (4 and 8 bits move from the fused kernel to the two-kernel path), each with just enough 256 x 256 tiles
# for those paths to be taken; and the shapes on either side of what the eight-rows matvecs take.
_LARGE_BORDERS = [
    # M, K, N, bits, gs, transpose
    (1023, 512, 8456, 5, 64, True), (1024, 512, 8456, 5, 64, True), (1025, 384, 8712, 3, 32, True),
    (1024, 640, 8448, 6, 128, True), (2047, 512, 3848, 4, 64, True), (2048, 512, 3848, 4, 64, True),
    (2049, 384, 3848, 8, 32, True), (2048, 256, 4104, 8, 128, True), (1500, 512, 8456, 4, 64, True),
    (2048, 512, 3840, 6, 64, True), (1024, 512, 8440, 3, 64, True),
    # untransposed: x [M, N] @ dequant(w [N, K]) -> [M, K]
    (1023, 8448, 512, 4, 64, False), (1024, 8448, 512, 4, 64, False), (1025, 8512, 384, 8, 32, False),
    (2049, 3872, 512, 4, 32, False), (2048, 3840, 640, 8, 128, False), (2048, 3840, 576, 4, 64, False),
    (1024, 8448, 512, 5, 64, False),
]


@pytest.mark.parametrize("case", _LARGE_BORDERS, ids=lambda c: "M%d-K%d-N%d-w%d-g%d-%s" % c)
def test_large_m_borders_against_oracle(oracle, case):
    import mflux_amd
    from gpu_util import to_dev, u32_to_dev

    o = oracle
    M, K, N, bits, gs, transpose = case
    print(case, flush=True)
    if transpose:
        args = _case(o, 700 + M % 97 + bits, M, K, N, bits, gs=gs, with_bias=bool(M % 2))
        _assert_close(_run(o, *args, bits, gs), _ref(o, *args, bits, gs))
        return
    w = o.f32_to_bf16_bits(seeded(800 + bits, 1, (N, K), 0.02))
    wq, s, b = o.c_quantize(w, o.BF16, gs, bits)
    g = o.f32_to_bf16_bits(seeded(800 + bits, 5, (M, N), 1.0))
    ref = o.bf16_bits_to_f32(g).astype(np.float64) @ o.dequantize_exact(wq, s, b, o.BF16, gs, bits)
    y = mflux_amd.quantized_matmul(to_dev(g, o.BF16), u32_to_dev(wq), to_dev(s, o.BF16), to_dev(b, o.BF16),
                                   transpose=False, group_size=gs, bits=bits)
    assert tuple(y.shape) == (M, K)
    _assert_close(y, ref)


def _matvec_border_cases():
    rng = np.random.default_rng(20241125)
    cases = []
    for i in range(24):
        M = int(rng.choice([1, 2, 3, 4, 5]))
        K = int(rng.choice([1024, 2048, 3072, 4096, 5120, 1088, 960]))
        N = int(rng.choice([8, 72, 100, 2312, 20, 9224]))
        bits = int(rng.choice([4, 8]))
        gs = int(rng.choice([64, 64, 64, 32, 128]))
        if K % gs:
            K = K // gs * gs
        cases.append((i, M, K, N, bits, gs))
    return cases


@pytest.mark.parametrize("case", _matvec_border_cases(), ids=lambda c: "case%d-M%d-K%d-N%d-w%d-g%d" % c)
def test_matvec_borders_against_oracle(oracle, case):
    """Shapes on both sides of what the eight-rows matvecs take (K in steps of 1024
    up to 4096, groups of 64, N a multiple of 8, one to four rows): whichever
    kernel takes the call, the product holds the tolerance."""
    o = oracle
    i, M, K, N, bits, gs = case
    args = _case(o, 900 + i, M, K, N, bits, gs=gs, with_bias=bool(i % 2))
    x_norm = np.linalg.norm(o.bf16_bits_to_f32(args[0]).astype(np.float64), axis=-1, keepdims=True)
    _assert_close(_run(o, *args, bits, gs), _ref(o, *args, bits, gs), row_floor=0.02 * x_norm)


def test_torch_ops_and_ctypes_routes_agree_bit_for_bit(oracle):
    """The two ways into libmfq -- torch.ops.mfq (what mflux_amd.core uses) and the
    C ABI through ctypes -- run the same kernels on the same stream: quantize,
    dequantize and the product (matvec, medium-M with a K split, large-M) come
    out bit-identical."""
    from gpu_util import to_dev
    from mflux_amd import _lib

    o = oracle
    lib, ops = _lib.load(), _lib.ops()
    stream = torch.cuda.current_stream().cuda_stream
    for M, K, N, bits in ((1, 3072, 512, 8), (300, 2048, 1024, 4), (700, 512, 1536, 8)):
        x = to_dev(o.f32_to_bf16_bits(seeded(81, 0, (M, K), 1.0)), o.BF16)
        w = to_dev(o.f32_to_bf16_bits(seeded(81, 1, (N, K), 0.02)), o.BF16)
        bias = to_dev(o.f32_to_bf16_bits(seeded(81, 2, (N,), 0.02)), o.BF16)
        wq, s, b = ops.quantize_affine(w, 64, bits)
        wq_c = torch.empty_like(wq)
        s_c, b_c = torch.empty_like(s), torch.empty_like(b)
        assert lib.mfq_quantize_affine(w.data_ptr(), _lib.BF16, N, K, 64, bits, wq_c.data_ptr(), s_c.data_ptr(),
                                       b_c.data_ptr(), stream) == 0
        assert torch.equal(wq.view(torch.int32), wq_c.view(torch.int32))
        assert torch.equal(s.view(torch.int16), s_c.view(torch.int16)) and torch.equal(b.view(torch.int16), b_c.view(torch.int16))
        d = ops.dequantize_affine(wq, s, b, 64, bits, torch.bfloat16)
        d_c = torch.empty_like(d)
        assert lib.mfq_dequantize_affine(wq.data_ptr(), s.data_ptr(), b.data_ptr(), _lib.BF16, N, K, 64, bits,
                                         d_c.data_ptr(), _lib.BF16, stream) == 0
        assert torch.equal(d.view(torch.int16), d_c.view(torch.int16))
        y, ok = ops.qmm_t(x, wq, s, b, bias, 64, bits, torch.bfloat16, None, None)
        assert ok
        need = lib.mfq_qmm_t_workspace_bytes(M, K, N, 64, bits)
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
        y_c = torch.empty_like(y)
        assert lib.mfq_qmm_t_ws(x.data_ptr(), _lib.BF16, M, K, wq.data_ptr(), s.data_ptr(), b.data_ptr(), _lib.BF16,
                                bias.data_ptr(), N, 64, bits, y_c.data_ptr(), _lib.BF16, ws.data_ptr(), need, stream) == 0
        torch.cuda.synchronize()
        assert torch.equal(y.view(torch.int16), y_c.view(torch.int16)), (M, K, N, bits)
