"""GPU parity of the GEMM epilogues (mfq_qmm_t_epilogue): what mflux does to a
quantized linear's output next -- gelu_approx, residual + gate * y, SwiGLU --
inside the kernel that writes y.  Against float64 (the exact product on the
MLX-format operands, then the operation): the product's tolerance, 1e-2 of the
output row's largest magnitude, plus 2^-8 (half a bfloat16 ulp at worst) for
every further operation, since the reference rounds to bfloat16 after each of
them and so does the kernel.  The sharper check is the second one: against the
same operations applied to the plain call's result, which rounds at the same
points -- bit for bit where only roundings are involved, within one or two
units in the last place where the hardware exponential and reciprocal are."""
import numpy as np
import pytest
import torch

from conftest import seeded

pytestmark = pytest.mark.gpu

TOL = 1e-2
ULP = 2.0 ** -8  # one more rounding to bfloat16, relative to the value

# (M, K, N, bits, gs): which kernel takes the shape
SHAPES = [
    (2304, 512, 4096, 4, 64),    # 256 x 256 tiles, whole tiles only
    (4400, 1024, 3840, 8, 64),   # 256 x 256 tiles, the short last round cut along K (second kernel)
    (300, 512, 1024, 4, 64),     # 128-column tiles
    (512, 3072, 3072, 4, 64),    # 128-column tiles cut along K (second kernel)
    (200, 1024, 640, 5, 128),    # 5-bit stream
    (77, 96, 128, 8, 32),        # K % 64 == 32
    (100, 256, 192, 4, 64),      # 128-row tiles
]


def _operands(o, cfg, M, K, N, bits, gs):
    from gpu_util import to_dev, u32_to_dev

    x = o.f32_to_bf16_bits(seeded(cfg, 0, (M, K), 1.0))
    w = o.f32_to_bf16_bits(seeded(cfg, 1, (N, K), 0.02 if K >= 512 else 0.08))
    bias = o.f32_to_bf16_bits(seeded(cfg, 2, (N,), 0.02))
    wq, s, b = o.c_quantize(w, o.BF16, gs, bits)
    y64 = o.quantized_matmul_f64(o.bf16_bits_to_f32(x).astype(np.float64), wq, s, b, o.BF16, gs, bits,
                                 bias_f64=o.bf16_bits_to_f32(bias).astype(np.float64))
    dev = (to_dev(x, o.BF16), u32_to_dev(wq), to_dev(s, o.BF16), to_dev(b, o.BF16), to_dev(bias, o.BF16))
    return dev, y64


def _close(y, ref, tol=TOL):
    got = y.detach().double().cpu().numpy()
    assert got.shape == ref.shape
    err = np.abs(got - ref).max(axis=-1) / np.maximum(np.abs(ref).max(axis=-1), 1e-30)
    assert err.max() <= tol, f"max |err| / ||row||inf = {err.max():.4g}"


def _ulps_apart(a, b):
    """largest difference of two bfloat16 tensors in units of the larger one's last place; values below 2^-8
    (of rows whose largest magnitude is about 1) count as 2^-8: down its negative tail gelu_approx is
    x * (1 + tanh(.)) with 1 + tanh cancelling in float32 in one evaluation and x * sigmoid(.) in the other"""
    a32, b32 = a.float(), b.float()
    ulp = torch.maximum(a32.abs(), b32.abs()).clamp_min(2.0 ** -8) * 2.0 ** -7
    return float(((a32 - b32).abs() / ulp).max())


def _gelu64(v):
    return 0.5 * v * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (v + 0.044715 * v ** 3)))


def _fused_ran(M, K, N, bits, gs, name, dev, **kw):
    """the C ABI's own answer for this shape: 0 (a kernel fused it) or MFQ_EUNSUPPORTED"""
    from mflux_amd import _lib

    ops = _lib.ops()
    x, wq, s, b, bias = dev
    y, ok = ops.qmm_t_epilogue(x, wq, s, b, bias, gs, bits, kw["kind"], kw.get("gate"), kw.get("residual"),
                               kw.get("act_from", 0))
    return ok


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "M%d-K%d-N%d-w%d-g%d" % s)
def test_gelu_epilogue(oracle, shape):
    import mflux_amd

    M, K, N, bits, gs = shape
    print(f"gelu {shape}", flush=True)
    dev, y64 = _operands(oracle, 95, M, K, N, bits, gs)
    x, wq, s, b, bias = dev
    for act_from in (0, N // 2 // 8 * 8):
        assert _fused_ran(M, K, N, bits, gs, "gelu", dev, kind=1, act_from=act_from)
        y = mflux_amd.quantized_matmul_epilogue(x, wq, s, b, epilogue="gelu", group_size=gs, bits=bits, bias=bias,
                                                act_from=act_from)
        ref = y64.copy()
        ref[:, act_from:] = _gelu64(ref[:, act_from:])
        _close(y, ref, tol=TOL + ULP)
        plain = mflux_amd.quantized_matmul(x, wq, s, b, group_size=gs, bits=bits, bias=bias)
        assert torch.equal(y[:, :act_from].view(torch.int16), plain[:, :act_from].view(torch.int16))
        assert _ulps_apart(y[:, act_from:], mflux_amd.gelu_approx(plain[:, act_from:])) <= 1.01


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "M%d-K%d-N%d-w%d-g%d" % s)
def test_gate_residual_epilogue(oracle, shape):
    import mflux_amd
    from gpu_util import to_dev

    o = oracle
    M, K, N, bits, gs = shape
    print(f"gate_residual {shape}", flush=True)
    dev, y64 = _operands(o, 96, M, K, N, bits, gs)
    x, wq, s, b, bias = dev
    gate_h = o.f32_to_bf16_bits(seeded(96, 3, (N,), 1.0))
    res_h = o.f32_to_bf16_bits(seeded(96, 4, (M, N), 1.0))
    gate, res = to_dev(gate_h, o.BF16), to_dev(res_h, o.BF16)
    assert _fused_ran(M, K, N, bits, gs, "gate_residual", dev, kind=2, gate=gate, residual=res)
    guard = torch.full((4, N), 7.0, device="cuda", dtype=torch.bfloat16)
    y = mflux_amd.quantized_matmul_epilogue(x, wq, s, b, epilogue="gate_residual", group_size=gs, bits=bits, bias=bias,
                                            gate=gate.reshape(1, N), residual=res)
    ref = o.bf16_bits_to_f32(res_h).astype(np.float64) + o.bf16_bits_to_f32(gate_h).astype(np.float64) * y64
    _close(y, ref, tol=TOL + 2 * ULP)
    # the same roundings as the separate operations: bit for bit
    plain = mflux_amd.quantized_matmul(x, wq, s, b, group_size=gs, bits=bits, bias=bias)
    assert torch.equal(y.view(torch.int16), (res + gate * plain).view(torch.int16))
    assert bool((guard == 7.0).all())


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "M%d-K%d-N%d-w%d-g%d" % s)
def test_swiglu_epilogue(oracle, shape):
    import mflux_amd

    M, K, N, bits, gs = shape
    print(f"swiglu {shape}", flush=True)
    dev, y64 = _operands(oracle, 97, M, K, N, bits, gs)
    x, wq, s, b, bias = dev
    assert _fused_ran(M, K, N, bits, gs, "swiglu", dev, kind=3)
    guard = torch.full((4, N // 2), 7.0, device="cuda", dtype=torch.bfloat16)
    y = mflux_amd.quantized_matmul_epilogue(x, wq, s, b, epilogue="swiglu", group_size=gs, bits=bits, bias=bias)
    assert tuple(y.shape) == (M, N // 2)
    blocks = y64.reshape(M, N // 64, 2, 32)
    g, u = blocks[:, :, 0, :], blocks[:, :, 1, :]
    ref = (g / (1.0 + np.exp(-g)) * u).reshape(M, N // 2)
    _close(y, ref, tol=2 * TOL + 3 * ULP)  # two values that each carry the product's tolerance; sigmoid, x * s, * u
    plain = mflux_amd.quantized_matmul(x, wq, s, b, group_size=gs, bits=bits, bias=bias)
    from mflux_amd.core import swiglu_unstack
    assert _ulps_apart(y, swiglu_unstack(plain)) <= 2.01  # the sigmoid's last place can move the product's
    assert bool((guard == 7.0).all())


def test_epilogue_module_helpers_and_composed_paths(oracle):
    """nn.gelu_linear / gate_residual_linear / stack_gate_up + swiglu_linear on
    quantized layers, and the calls no kernel fuses (a few rows, float32 x, a
    float layer): the same values from the composed form."""
    import mflux_amd
    from mflux_amd import nn as qnn

    torch.manual_seed(11)
    K, H = 256, 192
    w1 = qnn.Linear(K, H, bias=False, device="cuda", dtype=torch.bfloat16)
    w3 = qnn.Linear(K, H, bias=False, device="cuda", dtype=torch.bfloat16)
    q1, q3 = w1.to_quantized(bits=8), w3.to_quantized(bits=8)
    stacked = qnn.stack_gate_up(q1, q3)
    assert tuple(stacked.weight.shape) == (2 * H, K * 8 // 32)
    for M in (200, 4):
        x = torch.randn(M, K, device="cuda").to(torch.bfloat16)
        want = mflux_amd.silu(q1(x)) * q3(x)   # feed_forward.py:13 as the reference writes it
        got = qnn.swiglu_linear(stacked, x)
        assert _ulps_apart(got, want) <= 2.01, M
        gate = torch.randn(H, device="cuda").to(torch.bfloat16)
        res = torch.randn(M, H, device="cuda").to(torch.bfloat16)
        assert torch.equal(qnn.gate_residual_linear(q1, x, gate, res), res + gate * q1(x))
        assert _ulps_apart(qnn.gelu_linear(q1, x), mflux_amd.gelu_approx(q1(x))) <= 1.01
        assert torch.equal(qnn.gate_residual_linear(w1, x, gate, res), res + gate * w1(x))  # float layer: composed
        # one gate vector per batch entry, expanded over the sequence as the reference does
        # (joint_transformer_block.py:84-90: mx.expand_dims(gate, 1)): [B, N] and [B, 1, N] next to x of [B, S, K]
        xb = torch.stack([x, x.flip(0)])
        resb = torch.stack([res, res.flip(0)])
        gates = torch.stack([gate.reshape(-1), gate.reshape(-1).flip(0)])
        want = torch.stack([resb[i] + gates[i] * q1(xb[i]) for i in range(2)])   # (per entry: the same kernel as above)
        assert torch.equal(qnn.gate_residual_linear(q1, xb, gates, resb), want)
        assert torch.equal(qnn.gate_residual_linear(q1, xb, gates[:, None, :], resb), want)
        with pytest.raises(ValueError, match="per batch entry"):
            qnn.gate_residual_linear(q1, xb, gates[:, :8], resb)
    x32 = torch.randn(40, K, device="cuda")
    y = mflux_amd.quantized_matmul_epilogue(x32, q1.weight, q1.scales, q1.biases, epilogue="gelu", bits=8)
    assert y.dtype == torch.float32
    assert torch.allclose(y, mflux_amd.gelu_approx(mflux_amd.quantized_matmul(x32, q1.weight, q1.scales, q1.biases, bits=8)))
    with pytest.raises(ValueError, match="unknown epilogue"):
        mflux_amd.quantized_matmul_epilogue(x32, q1.weight, q1.scales, q1.biases, epilogue="relu", bits=8)
    with pytest.raises(ValueError, match="needs gate and residual"):
        mflux_amd.quantized_matmul_epilogue(x32, q1.weight, q1.scales, q1.biases, epilogue="gate_residual", bits=8)
