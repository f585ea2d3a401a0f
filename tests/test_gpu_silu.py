"""GPU parity: the adaLN modulation call linear(silu(x)) as one kernel
(mfq_qmv_silu, reached through mflux_amd.silu_quantized_matmul) against the
oracle's silu (two roundings in the 16-bit type) followed by the float64
matmul on MLX-format operands.

Tolerance of this path: max |y - y_ref| <= 1e-2 * max|y_ref row|.
"""
import numpy as np
import pytest
import torch

from conftest import seeded

pytestmark = pytest.mark.gpu

TOL = 1e-2


def _operands(o, cfg, K, N, bits, gs, dtype, with_bias, x_std=2.0):
    x = o._from_f32(seeded(cfg, 0, (1, K), x_std), dtype)
    w = o._from_f32(seeded(cfg, 1, (N, K), 0.02), dtype)
    bias = o._from_f32(seeded(cfg, 2, (N,), 0.02), dtype) if with_bias else None
    wq, s, b = o.c_quantize(w, dtype, gs, bits)
    return x, wq, s, b, bias


def _dev(o, x, wq, s, b, bias, dtype):
    from gpu_util import to_dev, u32_to_dev

    return (to_dev(x, dtype), u32_to_dev(wq), to_dev(s, dtype), to_dev(b, dtype),
            None if bias is None else to_dev(bias, dtype))


def _ref(o, x, wq, s, b, bias, dtype, gs, bits):
    xs = o._to_f32(o.silu_bits(x, dtype), dtype).astype(np.float64)
    bf = None if bias is None else o._to_f32(bias, dtype).astype(np.float64)
    return o.quantized_matmul_f64(xs, wq, s, b, dtype, gs, bits, bias_f64=bf)


def _worst(y: torch.Tensor, ref: np.ndarray) -> float:
    got = y.detach().to(torch.float64).cpu().numpy()
    assert got.shape == ref.shape
    return float((np.abs(got - ref) / np.abs(ref).max(axis=-1, keepdims=True)).max())


@pytest.mark.parametrize("with_bias", [True, False])
@pytest.mark.parametrize("dtype_name", ["bf16", "f16"])
@pytest.mark.parametrize("bits,gs,K", [(8, 64, 3072), (4, 64, 3072), (8, 64, 1088), (4, 128, 2048), (8, 32, 3072),
                                       (4, 64, 6144), (8, 64, 6144)])
def test_silu_matvec_vs_f64(oracle, bits, gs, K, dtype_name, with_bias):
    import mflux_amd

    o = oracle
    dtype = o.BF16 if dtype_name == "bf16" else o.F16
    ops = _operands(o, 31, K, 1024 + 24, bits, gs, dtype, with_bias)
    x, wq, s, b, bias = _dev(o, *ops, dtype)
    y = mflux_amd.silu_quantized_matmul(x, wq, s, b, group_size=gs, bits=bits, bias=bias)
    torch.cuda.synchronize()
    assert y.shape == (1, 1024 + 24) and y.dtype == x.dtype
    assert _worst(y, _ref(o, *ops, dtype, gs, bits)) <= TOL


@pytest.mark.parametrize("M", [2, 3, 4])
@pytest.mark.parametrize("bits,dtype_name,K", [(8, "bf16", 3072), (4, "bf16", 3072), (8, "f16", 1024), (4, "f16", 4096)])
def test_silu_matvec_up_to_four_rows(oracle, bits, dtype_name, K, M):
    """Two to four activation rows (a batch): the activation inside the four-rows kernel."""
    import mflux_amd
    from gpu_util import to_dev

    o = oracle
    dtype = o.BF16 if dtype_name == "bf16" else o.F16
    N = 1024 + 24
    ops = _operands(o, 37, K, N, bits, 64, dtype, True)
    xm = o._from_f32(seeded(37, 5, (M, K), 2.0) * np.float32([[1.0], [0.01], [30.0], [3.0]][:M]), dtype)
    _, wq, s, b, bias = _dev(o, *ops, dtype)
    y = mflux_amd.silu_quantized_matmul(to_dev(xm, dtype), wq, s, b, group_size=64, bits=bits, bias=bias)
    torch.cuda.synchronize()
    assert y.shape == (M, N)
    ref = _ref(o, xm, *ops[1:], dtype, 64, bits)
    assert _worst(y, ref) <= TOL
    # and against the composition: the same kernel behind a separate activation
    want = mflux_amd.quantized_matmul(mflux_amd.silu(to_dev(xm, dtype)), wq, s, b, group_size=64, bits=bits, bias=bias)
    assert float((y.double() - want.double()).abs().max() / want.double().abs().max()) <= 2e-3


def test_silu_matvec_adaln_full_size(oracle):
    """FLUX.1 double-block norm1: 3072 -> 18432, 8 bits, through the C ABI entry point itself."""
    from mflux_amd import _lib

    o = oracle
    K, N = 3072, 18432
    ops = _operands(o, 32, K, N, 8, 64, o.BF16, True, x_std=1.0)
    x, wq, s, b, bias = _dev(o, *ops, o.BF16)
    y = torch.empty((1, N), dtype=torch.bfloat16, device="cuda")
    rc = _lib.load().mfq_qmv_silu(x.data_ptr(), _lib.BF16, 1, K, wq.data_ptr(), s.data_ptr(), b.data_ptr(), _lib.BF16,
                                  bias.data_ptr(), N, 64, 8, y.data_ptr(), _lib.BF16,
                                  torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert _worst(y, _ref(o, *ops, o.BF16, 64, 8)) <= TOL


@pytest.mark.parametrize("dtype_name", ["bf16", "f16"])
def test_silu_values_through_a_unit_weight(oracle, dtype_name):
    """Codes 1 on the diagonal, 0 elsewhere, scale 1, bias 0: y[n] is silu(x)[n]
    up to the kernel's 15-bit fixed point (2^-15 of the row's largest magnitude)
    and the rounding of y, which isolates the activation's values."""
    import mflux_amd
    from gpu_util import to_dev, u32_to_dev

    o = oracle
    dtype = o.BF16 if dtype_name == "bf16" else o.F16
    K = N = 1024
    x = o._from_f32(seeded(33, 0, (1, K), 2.5), dtype)
    n = np.arange(N)
    wq = np.zeros((N, K // 4), dtype=np.uint32)
    wq[n, n // 4] = np.uint32(1) << (8 * (n % 4)).astype(np.uint32)
    one = o._from_f32(np.ones((N, K // 64), np.float32), dtype)
    zero = o._from_f32(np.zeros((N, K // 64), np.float32), dtype)
    y = mflux_amd.silu_quantized_matmul(to_dev(x, dtype), u32_to_dev(wq), to_dev(one, dtype), to_dev(zero, dtype),
                                        group_size=64, bits=8)
    torch.cuda.synchronize()
    got = y.to(torch.float64).cpu().numpy().reshape(-1)
    ref = o._to_f32(o.silu_bits(x, dtype), dtype).astype(np.float64).reshape(-1)
    ulp = 2.0 ** (-8 if dtype == o.BF16 else -11)
    bound = 2.0 ** -14 * np.abs(ref).max() + 2 * ulp * np.abs(ref)   # fixed point + rounding of y + one ulp of silu
    assert np.all(np.abs(got - ref) <= bound)
    # and it is the activation, not the identity
    xf = o._to_f32(x, dtype).astype(np.float64).reshape(-1)
    assert np.abs(got - xf).max() > 0.25


@pytest.mark.parametrize("bits", [4, 8])
def test_silu_fused_against_composition(oracle, bits):
    """The fused call against silu as a pass of its own in front of the same
    matvec: the two sigmoids may round a value of x the other way now and then,
    nothing else differs."""
    import mflux_amd

    o = oracle
    ops = _operands(o, 34, 3072, 2048, bits, 64, o.BF16, True)
    x, wq, s, b, bias = _dev(o, *ops, o.BF16)
    fused = mflux_amd.silu_quantized_matmul(x, wq, s, b, group_size=64, bits=bits, bias=bias)
    composed = mflux_amd.quantized_matmul(mflux_amd.silu(x), wq, s, b, group_size=64, bits=bits, bias=bias)
    torch.cuda.synchronize()
    a, c = fused.double(), composed.double()
    assert float((a - c).abs().max() / c.abs().max()) <= 2e-3


def test_silu_calls_without_a_fused_kernel_compose(oracle):
    """More than four rows, rows longer than the fused kernels take, odd bit
    widths and float32 x run silu as its own pass: identical to the composition."""
    import mflux_amd

    o = oracle
    for M, K, bits in ((5, 3072, 8), (1, 8192, 8), (1, 3072, 5), (3, 8192, 4)):
        ops = _operands(o, 35, K, 256, bits, 64, o.BF16, True)
        x, wq, s, b, bias = _dev(o, *ops, o.BF16)
        x = x.expand(M, K).contiguous() * torch.arange(1, M + 1, device="cuda", dtype=torch.bfloat16)[:, None]
        y = mflux_amd.silu_quantized_matmul(x, wq, s, b, group_size=64, bits=bits, bias=bias)
        want = mflux_amd.quantized_matmul(mflux_amd.silu(x), wq, s, b, group_size=64, bits=bits, bias=bias)
        assert torch.equal(y, want)
    ops = _operands(o, 35, 3072, 256, 8, 64, o.BF16, False)
    x, wq, s, b, _ = _dev(o, *ops, o.BF16)
    y = mflux_amd.silu_quantized_matmul(x.float(), wq, s, b, group_size=64, bits=8)
    assert y.dtype == torch.float32
    assert torch.equal(y, mflux_amd.quantized_matmul(mflux_amd.silu(x.float()), wq, s, b, group_size=64, bits=8))


def test_silu_not_finite_input_gives_nan(oracle):
    import mflux_amd

    o = oracle
    ops = _operands(o, 36, 3072, 128, 8, 64, o.BF16, False)
    x, wq, s, b, _ = _dev(o, *ops, o.BF16)
    x = x.clone()
    x[0, 17] = float("inf")
    y = mflux_amd.silu_quantized_matmul(x, wq, s, b, group_size=64, bits=8)
    assert bool(torch.isnan(y).all())
    x[0, 17] = -200.0   # the sigmoid is 0 there and the product -0: finite everywhere
    y = mflux_amd.silu_quantized_matmul(x, wq, s, b, group_size=64, bits=8)
    assert bool(torch.isfinite(y).all())


def test_silu_linear_wrapper(oracle):
    """nn.silu_linear: fused on a QuantizedLinear, the composition on anything else;
    leading dimensions of x are kept."""
    import mflux_amd
    from mflux_amd import nn as qnn

    torch.manual_seed(5)
    lin = qnn.Linear(3072, 512, bias=True, device="cuda", dtype=torch.bfloat16)
    q = lin.to_quantized(64, 8)
    x = (torch.randn(1, 1, 3072, device="cuda") * 2).to(torch.bfloat16)
    y = qnn.silu_linear(q, x)
    assert y.shape == (1, 1, 512)
    want = q(mflux_amd.silu(x))
    assert float((y.double() - want.double()).abs().max() / want.double().abs().max()) <= 2e-3
    y_float = qnn.silu_linear(lin, x)
    assert torch.equal(y_float, lin(mflux_amd.silu(x)))
    x.requires_grad_(True)   # gradients: the composed, differentiable form
    qnn.silu_linear(q, x).float().sum().backward()
    assert x.grad is not None and bool(torch.isfinite(x.grad).all())


def test_modulation_linears_of_several_blocks_as_one_call(oracle):
    """The modulation linears of all blocks take the same silu(temb): stacked
    along N (sharing storage with the layers) they give, in one call, bit for
    bit what each layer gives on its own, since a row's result does not depend
    on how rows are dealt out."""
    import mflux_amd
    from mflux_amd import nn as qnn

    torch.manual_seed(6)
    layers = [qnn.Linear(3072, n, bias=True, device="cuda", dtype=torch.bfloat16).to_quantized(64, 8)
              for n in (18432, 18432, 9216, 6144)]
    for layer in layers:
        layer.bias.normal_(0, 0.02)
    temb = (torch.randn(1, 3072, device="cuda") * 2).to(torch.bfloat16)
    alone = [qnn.silu_linear(layer, temb) for layer in layers]
    bank = qnn.concat_quantized(layers, share_storage=True)
    parts = qnn.silu_linear(bank, temb).split([layer.output_dims for layer in layers], dim=-1)
    for part, ref, layer in zip(parts, alone, layers):
        assert torch.equal(part, ref)
        assert torch.equal(qnn.silu_linear(layer, temb), ref)     # the layers still work, now as views of the bank
