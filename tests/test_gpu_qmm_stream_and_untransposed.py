"""GPU parity of the two GEMM kernels that complete the product: 3-, 5- and
6-bit weights against more than one activation row (MLX's 3- and 5-byte packs
cut out of the bit stream inside the 128-column-tile kernel), and the product
with the weight not transposed (transpose=False, the input gradient of a
quantized linear).  Both against the float64 product on the exactly dequantized
weight, tolerance 1e-2 of the output row's largest magnitude."""
import numpy as np
import pytest
import torch

from conftest import seeded

pytestmark = pytest.mark.gpu

TOL = 1e-2


def _close(y, ref, tol=TOL):
    got = y.detach().double().cpu().numpy()
    assert got.shape == ref.shape
    err = np.abs(got - ref).max(axis=-1) / np.maximum(np.abs(ref).max(axis=-1), 1e-30)
    assert err.max() <= tol, f"max |err| / ||row||inf = {err.max():.4g}"


def _weights(o, cfg, N, K, bits, gs, dtype=None):
    dtype = o.BF16 if dtype is None else dtype
    w = seeded(cfg, 1, (N, K), 0.02)
    ws = o.f32_to_bf16_bits(w) if dtype == o.BF16 else w.astype(np.float16).view(np.uint16)
    return o.c_quantize(ws, dtype, gs, bits)


@pytest.mark.parametrize("bits", [3, 5, 6])
@pytest.mark.parametrize("M,K,N,gs", [
    (2, 3072, 200, 64),        # two rows: 128-row tiles
    (17, 512, 1000, 64),
    (128, 2048, 264, 128),
    (129, 1024, 136, 32),      # 256-row tiles: half of the threads dequantise
    (300, 3072, 3072, 64),     # few tiles, long K: cut along K with the workspace
    (1100, 4096, 520, 64),
    (40, 2176, 17, 64),        # N below one tile, K = 34 steps
    (77, 96, 40, 32),          # K % 64 == 32: the last step is half zeros
    (513, 1056, 72, 32),
])
def test_stream_bits_gemm(oracle, bits, M, K, N, gs):
    import mflux_amd
    from gpu_util import to_dev, u32_to_dev

    o = oracle
    print(f"bits={bits} M={M} K={K} N={N} gs={gs}", flush=True)
    x = o.f32_to_bf16_bits(seeded(91, 0, (M, K), 1.0))
    bias = o.f32_to_bf16_bits(seeded(91, 2, (N,), 0.02))
    wq, s, b = _weights(o, 91, N, K, bits, gs)
    ref = o.quantized_matmul_f64(o.bf16_bits_to_f32(x).astype(np.float64), wq, s, b, o.BF16, gs, bits,
                                 bias_f64=o.bf16_bits_to_f32(bias).astype(np.float64))
    guard = torch.full((4, N), 7.0, device="cuda", dtype=torch.bfloat16)
    y = mflux_amd.quantized_matmul(to_dev(x, o.BF16), u32_to_dev(wq), to_dev(s, o.BF16), to_dev(b, o.BF16),
                                   group_size=gs, bits=bits, bias=to_dev(bias, o.BF16))
    assert y.dtype == torch.bfloat16
    _close(y, ref)
    y32 = mflux_amd.quantized_matmul(to_dev(x, o.BF16).float(), u32_to_dev(wq), to_dev(s, o.BF16), to_dev(b, o.BF16),
                                     group_size=gs, bits=bits, bias=to_dev(bias, o.BF16))
    assert y32.dtype == torch.float32
    _close(y32, ref, tol=5e-3)
    assert bool((guard == 7.0).all())


@pytest.mark.parametrize("bits", [3, 5, 6])
def test_stream_bits_gemm_one_hot_rows_are_dequantised_weight_rows(oracle, bits):
    """x = one-hot rows: y[m, :] is column k_m of the dequantised weight, rounded
    once -- pins the position of every code in the bit stream end to end."""
    import mflux_amd
    from gpu_util import raw, to_dev, u32_to_dev

    o = oracle
    M, K, N = 96, 192, 130
    wq, s, b = _weights(o, 92, N, K, bits, 64)
    hot = (np.arange(M) * 2 + 1) % K
    x = np.zeros((M, K), dtype=np.float32)
    x[np.arange(M), hot] = 1.0
    y = mflux_amd.quantized_matmul(to_dev(o.f32_to_bf16_bits(x), o.BF16), u32_to_dev(wq), to_dev(s, o.BF16),
                                   to_dev(b, o.BF16), group_size=64, bits=bits)
    exact = o.dequantize_exact(wq, s, b, o.BF16, 64, bits)          # [N, K]
    expect = o.f32_to_bf16_bits(exact.astype(np.float32))[:, hot].T   # fma rounded once to bfloat16
    assert np.array_equal(raw(y), expect)


def test_stream_bits_gemm_f16_and_low_rank(oracle):
    import mflux_amd
    from gpu_util import raw

    o = oracle
    torch.manual_seed(4)
    for bits in (3, 5, 6):
        M, K, N, R = 200, 512, 320, 16
        x = torch.randn(M, K, device="cuda").to(torch.float16)
        w = (torch.randn(N, K, device="cuda") * 0.02).to(torch.float16)
        wq, s, b = mflux_amd.quantize(w, 64, bits)
        t = (torch.randn(M, R, device="cuda") * 0.5).to(torch.float16)
        bs = (torch.randn(N, R, device="cuda") * 0.05).to(torch.float16)
        y = mflux_amd.quantized_matmul(x, wq, s, b, bits=bits, low_rank=(t, bs))
        ref = o.quantized_matmul_f64(x.double().cpu().numpy(), raw(wq), raw(s), raw(b), o.F16, 64, bits)
        ref = ref + t.double().cpu().numpy() @ bs.double().cpu().numpy().T
        _close(y, ref)


@pytest.mark.parametrize("bits", [3, 4, 5, 6, 8])
@pytest.mark.parametrize("M,N,K,gs", [
    (1, 64, 64, 64),
    (40, 192, 512, 64),
    (129, 1000, 160, 32),      # N % 64 == 40: the last step is mostly zeros; K % 128 == 32: the last tile overhangs
    (300, 72, 3072, 128),
    (600, 3072, 1024, 64),
    (64, 203, 96, 32),         # N % 8 != 0: the host pads x and the weight
])
def test_untransposed_product(oracle, bits, M, N, K, gs):
    import mflux_amd
    from gpu_util import to_dev, u32_to_dev

    o = oracle
    print(f"bits={bits} M={M} N={N} K={K} gs={gs}", flush=True)
    wq, s, b = _weights(o, 93, N, K, bits, gs)
    g = o.f32_to_bf16_bits(seeded(93, 5, (M, N), 1.0))
    ref = o.bf16_bits_to_f32(g).astype(np.float64) @ o.dequantize_exact(wq, s, b, o.BF16, gs, bits)
    wd, sd, bd = u32_to_dev(wq), to_dev(s, o.BF16), to_dev(b, o.BF16)
    guard = torch.full((4, K), 7.0, device="cuda", dtype=torch.bfloat16)
    y = mflux_amd.quantized_matmul(to_dev(g, o.BF16), wd, sd, bd, transpose=False, group_size=gs, bits=bits)
    assert tuple(y.shape) == (M, K) and y.dtype == torch.bfloat16
    _close(y, ref)
    y32 = mflux_amd.quantized_matmul(to_dev(g, o.BF16).float().reshape(1, M, N), wd, sd, bd, transpose=False,
                                     group_size=gs, bits=bits)
    assert tuple(y32.shape) == (1, M, K) and y32.dtype == torch.float32
    _close(y32[0], ref, tol=5e-3)
    assert bool((guard == 7.0).all())


@pytest.mark.parametrize("bits", [3, 4, 5, 6, 8])
def test_untransposed_one_hot_rows_are_dequantised_weight_rows(oracle, bits):
    """x = one-hot rows: y[m, :] is row n_m of the dequantised weight, rounded
    once -- pins the transposing tile builder (row quads, column blocks, the
    funnel shift of the bit stream) end to end."""
    import mflux_amd
    from gpu_util import raw, to_dev, u32_to_dev

    o = oracle
    M, N, K = 150, 136, 416
    wq, s, b = _weights(o, 94, N, K, bits, 32)
    hot = (np.arange(M) * 3 + 2) % N
    x = np.zeros((M, N), dtype=np.float32)
    x[np.arange(M), hot] = 1.0
    y = mflux_amd.quantized_matmul(to_dev(o.f32_to_bf16_bits(x), o.BF16), u32_to_dev(wq), to_dev(s, o.BF16),
                                   to_dev(b, o.BF16), transpose=False, group_size=32, bits=bits)
    expect = o.f32_to_bf16_bits(o.dequantize_exact(wq, s, b, o.BF16, 32, bits).astype(np.float32))[hot]
    assert np.array_equal(raw(y), expect)


def test_untransposed_f16_and_full_size_gradient(oracle):
    """float16; and the gradient of FLUX.1's single-block linear1 at full size
    (g [4608, 21504] against the 4-bit weight [21504, 3072]): sampled rows
    against float64, every element against the dense product on the dequantized
    weight."""
    import mflux_amd
    from gpu_util import raw

    o = oracle
    torch.manual_seed(6)
    g = torch.randn(70, 264, device="cuda").to(torch.float16)
    w = (torch.randn(264, 320, device="cuda") * 0.02).to(torch.float16)
    wq, s, b = mflux_amd.quantize(w, 64, 8)
    y = mflux_amd.quantized_matmul(g, wq, s, b, transpose=False, bits=8)
    _close(y, g.double().cpu().numpy() @ o.dequantize_exact(raw(wq), raw(s), raw(b), o.F16, 64, 8))

    M, N, K = 4608, 21504, 3072
    g = torch.randn(M, N, device="cuda").to(torch.bfloat16)
    w = (torch.randn(N, K, device="cuda") * 0.02).to(torch.bfloat16)
    wq, s, b = mflux_amd.quantize(w, 64, 4)
    y = mflux_amd.quantized_matmul(g, wq, s, b, transpose=False, bits=4)
    rows = np.array([0, 255, 256, 2500, 4607])
    ref = o.bf16_bits_to_f32(raw(g[rows])).astype(np.float64) @ o.dequantize_exact(raw(wq), raw(s), raw(b), o.BF16, 64, 4)
    _close(y[rows], ref)
    dense = torch.matmul(g, mflux_amd.dequantize(wq, s, b, 64, 4)).float()
    assert float(((y.float() - dense).abs() / dense.abs().amax(dim=1, keepdim=True)).max()) <= 2 * TOL
