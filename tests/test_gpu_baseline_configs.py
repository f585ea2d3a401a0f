"""GPU parity at the full size of every benchmark configuration: the quantized
linears of FLUX.1 (to_q; the single-stream block), of a Z-Image block and of a
Qwen-Image double block, each at its own M, K, N, bit width and bias (the adaLN
modulation call of configuration 2, whose input is SiLU(temb), is
test_gpu_qmm.py::test_qmv_adaln_config_full).

Operands follow the benchmark's input convention: numpy default_rng(1000 *
config + tensor index), float32 normals (x ~ N(0, 1), W ~ N(0, 0.02), bias ~
N(0, 0.02)) rounded once to bfloat16 on the host, the same bit patterns for the
HIP path and the oracle.  Tensor indices: 10 * linear + (0: x, 1: W, 2: bias).

Checks per linear: the packed weight against the oracle's quantizer (bit for
bit, a band of rows), sampled output rows against the float64 product on the
MLX-format operands (tolerance 1e-2 of the row's largest magnitude), and every
element against a dense bfloat16 product on the dequantized weight from the BLAS
library (an independent GPU evaluation; twice the tolerance, since that product
rounds the weights a second time).
"""
import numpy as np
import pytest
import torch

from conftest import seeded

pytestmark = pytest.mark.gpu

TOL = 1e-2

# (id, config, linear index, M, K, N, bits, bias)
LINEARS = [
    ("cfg1_flux_to_q", 1, 0, 4096, 3072, 3072, 4, True),
    ("cfg3_flux_single_linear1", 3, 0, 4608, 3072, 21504, 4, True),
    ("cfg3_flux_single_linear2", 3, 1, 4608, 15360, 3072, 4, True),
    ("cfg3_flux_single_linear1_as_benchmarked_without_bias", 3, 0, 4608, 3072, 21504, 4, False),
    ("cfg4_zimage_attn_3840x3840", 4, 0, 4352, 3840, 3840, 8, False),
    ("cfg4_zimage_ffn_gate_up_3840x10240", 4, 1, 4352, 3840, 10240, 8, False),
    ("cfg4_zimage_ffn_down_10240x3840", 4, 2, 4352, 10240, 3840, 8, False),
    ("cfg5_qwen_img_attn_3072x3072", 5, 0, 6889, 3072, 3072, 4, True),
    ("cfg5_qwen_img_mlp_in_3072x12288", 5, 1, 6889, 3072, 12288, 4, True),
    ("cfg5_qwen_img_mlp_out_12288x3072", 5, 2, 6889, 12288, 3072, 4, True),
    ("cfg5_qwen_txt_attn_3072x3072", 5, 3, 256, 3072, 3072, 4, True),
    ("cfg5_qwen_txt_mlp_in_3072x12288", 5, 4, 256, 3072, 12288, 4, True),
    ("cfg5_qwen_txt_mlp_out_12288x3072", 5, 5, 256, 12288, 3072, 4, True),
    ("cfg5_qwen_modulation_3072x18432_m1", 5, 6, 1, 3072, 18432, 4, True),
]


def _operands(o, cfg, lin, M, K, N, with_bias):
    from gpu_util import to_dev

    x = o.f32_to_bf16_bits(seeded(cfg, 10 * lin + 0, (M, K), 1.0))
    w = o.f32_to_bf16_bits(seeded(cfg, 10 * lin + 1, (N, K), 0.02))
    bias = o.f32_to_bf16_bits(seeded(cfg, 10 * lin + 2, (N,), 0.02)) if with_bias else None
    return x, w, bias, to_dev(x, o.BF16), to_dev(w, o.BF16), None if bias is None else to_dev(bias, o.BF16)


@pytest.mark.parametrize("case", LINEARS, ids=[c[0] for c in LINEARS])
def test_baseline_linear_full_size(oracle, case):
    import mflux_amd
    from gpu_util import raw

    o = oracle
    name, cfg, lin, M, K, N, bits, with_bias = case
    print(f"{name}: M={M} K={K} N={N} bits={bits} bias={with_bias}", flush=True)
    x, w, bias, xd, wd, biasd = _operands(o, cfg, lin, M, K, N, with_bias)
    wq, s, b = mflux_amd.quantize(wd, 64, bits)
    band = slice(N // 2 - 32, N // 2 + 32)
    e_wq, e_s, e_b = o.c_quantize(w[band], o.BF16, 64, bits)
    assert np.array_equal(raw(wq[band]), e_wq) and np.array_equal(raw(s[band]), e_s) and np.array_equal(raw(b[band]), e_b)
    guard = torch.full((8, N), 7.0, device="cuda", dtype=torch.bfloat16)
    y = mflux_amd.quantized_matmul(xd, wq, s, b, group_size=64, bits=bits, bias=biasd)
    assert y.shape == (M, N) and y.dtype == torch.bfloat16
    rows = np.unique(np.clip(np.array([0, 1, 255, 256, M // 2, M - 257, M - 256, M - 2, M - 1]), 0, M - 1))
    ref = o.quantized_matmul_f64(o.bf16_bits_to_f32(x[rows]).astype(np.float64), raw(wq), raw(s), raw(b), o.BF16, 64,
                                 bits, bias_f64=None if bias is None else o.bf16_bits_to_f32(bias).astype(np.float64))
    got = y[torch.from_numpy(rows).cuda()].double().cpu().numpy()
    err = np.abs(got - ref).max(axis=1) / np.abs(ref).max(axis=1)
    assert err.max() <= TOL, f"{name}: max |err| / ||row||inf = {err.max():.4g}"
    dense = torch.matmul(xd, mflux_amd.dequantize(wq, s, b, 64, bits).t()).float()
    if biasd is not None:
        dense += biasd.float()
    row_inf = dense.abs().amax(dim=1, keepdim=True)
    assert float(((y.float() - dense).abs() / row_inf).max()) <= 2 * TOL
    assert bool((guard == 7.0).all())


def test_float32_activations_bound(oracle):
    """x in float32 that bfloat16 cannot represent (the input of to_out after
    rotary embeddings in float32, src/mflux/models/flux/model/flux_transformer/
    common/attention_utils.py:76-80): MLX promotes and computes in float32; this
    library rounds x to the scales' type for the matrix cores, as it rounds the
    dequantized weights, accumulates in float32 and returns float32.  Against the
    float64 product on the unrounded x the result stays within the tolerance of
    the path, and within 4e-3 of the row's largest magnitude at this shape
    (measured 1.2e-3: two operands with 2^-9 relative rounding each, K = 3072)."""
    import mflux_amd
    from gpu_util import raw, to_dev

    o = oracle
    M, K, N = 4096, 3072, 3072
    xf = seeded(1, 50, (M, K), 1.0)
    assert (o.bf16_bits_to_f32(o.f32_to_bf16_bits(xf)) != xf).mean() > 0.9, "x must not be bfloat16 values"
    wd = to_dev(o.f32_to_bf16_bits(seeded(1, 51, (N, K), 0.02)), o.BF16)
    biasd = to_dev(o.f32_to_bf16_bits(seeded(1, 52, (N,), 0.02)), o.BF16)
    wq, s, b = mflux_amd.quantize(wd, 64, 4)
    y = mflux_amd.quantized_matmul(torch.from_numpy(xf).cuda(), wq, s, b, group_size=64, bits=4, bias=biasd)
    assert y.dtype == torch.float32
    rows = np.array([0, 255, 1000, 2048, 4095])
    ref = o.quantized_matmul_f64(xf[rows].astype(np.float64), raw(wq), raw(s), raw(b), o.BF16, 64, 4,
                                 bias_f64=biasd.double().cpu().numpy())
    got = y[torch.from_numpy(rows).cuda()].double().cpu().numpy()
    err = np.abs(got - ref).max(axis=1) / np.abs(ref).max(axis=1)
    print(f"float32 x: max |err| / ||row||inf = {err.max():.3g}", flush=True)
    assert err.max() <= 4e-3
    # one row through the M = 1 kernel, whose fixed-point image of x is made from the rounded row as well
    y1 = mflux_amd.quantized_matmul(torch.from_numpy(xf[:1]).cuda(), wq, s, b, group_size=64, bits=4, bias=biasd)
    e1 = np.abs(y1.double().cpu().numpy() - ref[:1]).max() / np.abs(ref[0]).max()
    assert y1.dtype == torch.float32 and e1 <= 4e-3
