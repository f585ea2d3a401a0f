"""GPU parity: the matvec kernels that take eight weight rows at a time on the
int8 matrix instruction (csrc/qmv_oct.hip for 8-bit codes, csrc/qmv_oct4.hip
for 4-bit codes: groups of 64, one to four activation rows, K of 1024 .. 4096
in steps of 1024, N a multiple of 8) against the float64 oracle on MLX-format
operands, through the C ABI.

Tolerance of this path: max |y - y_ref| <= 1e-2 * max|y_ref row| per output
row; the cases with float32 output show how far inside it the kernel is.
"""
import numpy as np
import pytest
import torch

from conftest import seeded
from test_gpu_qmm import TOL, _assert_close, _case, _ref, _run

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("K", [1024, 2048, 3072, 4096])
@pytest.mark.parametrize("M", [1, 2, 3, 4])
def test_oct_vs_f64(oracle, K, M, bits):
    """Every K the kernel is built for (one to four 128-byte steps per
    wavefront), every number of activation rows, runs of blocks that are not
    whole trips of three (N = 8 * 53 rows: some workgroups get one block, some
    two), with the layer bias."""
    o = oracle
    args = _case(o, 61, M, K, 8 * 53 if K != 3072 else 8 * 530, bits)
    _assert_close(_run(o, *args, bits), _ref(o, *args, bits))


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("N", [8, 16, 24, 72, 8 * 257, 8 * 256 * 4 + 8, 8 * 256 * 12 + 16])
def test_oct_run_lengths(oracle, N, bits):
    """One block in all; fewer blocks than compute units; one, four and five
    blocks to a workgroup; and past twelve blocks to a compute unit, where the
    weight is cut into runs of nine blocks for as many workgroups as it takes."""
    o = oracle
    args = _case(o, 62, 2 if bits == 8 else 3, 1024, N, bits)
    _assert_close(_run(o, *args, bits), _ref(o, *args, bits))


@pytest.mark.parametrize("bits", [8, 4])
def test_oct_through_the_c_abi_f16_f32_no_bias(oracle, bits):
    """mfq_qmm_t through ctypes: float16 operands, float32 output, no bias; and
    bfloat16 with bias, bit for bit what the Python level returns."""
    import mflux_amd
    from gpu_util import to_dev, u32_to_dev
    from mflux_amd import _lib

    o = oracle
    lib = _lib.load()
    M, K, N = 3, 2048, 8 * 130
    x = o._from_f32(seeded(63, 0, (M, K), 1.0), o.F16)
    w = o._from_f32(seeded(63, 1, (N, K), 0.02), o.F16)
    wq, s, b = o.c_quantize(w, o.F16, 64, bits)
    xd, wd, sd, bd = to_dev(x, o.F16), u32_to_dev(wq), to_dev(s, o.F16), to_dev(b, o.F16)
    y = torch.empty(M, N, device="cuda", dtype=torch.float32)
    stream = torch.cuda.current_stream().cuda_stream
    rc = lib.mfq_qmm_t(xd.data_ptr(), _lib.F16, M, K, wd.data_ptr(), sd.data_ptr(), bd.data_ptr(), _lib.F16, None,
                       N, 64, bits, y.data_ptr(), _lib.F32, stream)
    assert rc == 0, rc
    torch.cuda.synchronize()
    ref = o.quantized_matmul_f64(o._to_f32(x, o.F16).astype(np.float64), wq, s, b, o.F16, 64, bits)
    _assert_close(y, ref, tol=2e-3)  # nothing is rounded to 16 bits on this path
    args = _case(o, 64, 4, 3072, 8 * 100, bits)
    y_py = _run(o, *args, bits)
    xb, wqb, sb, bb, bias = args
    xd, wd, sd, bd, biasd = (to_dev(xb, o.BF16), u32_to_dev(wqb), to_dev(sb, o.BF16), to_dev(bb, o.BF16),
                             to_dev(bias, o.BF16))
    y2 = torch.empty(4, 8 * 100, device="cuda", dtype=torch.bfloat16)
    rc = lib.mfq_qmm_t(xd.data_ptr(), _lib.BF16, 4, 3072, wd.data_ptr(), sd.data_ptr(), bd.data_ptr(), _lib.BF16,
                       biasd.data_ptr(), 8 * 100, 64, bits, y2.data_ptr(), _lib.BF16, stream)
    assert rc == 0, rc
    torch.cuda.synchronize()
    assert torch.equal(y2, y_py)
    _assert_close(y2, _ref(o, *args, bits), tol=TOL)


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("M", [1, 4])
def test_oct_one_hot_rows_return_weight_columns(oracle, M, bits):
    """One-hot activation rows return columns of the weight: every byte of a
    wavefront's 128-byte steps, both halves of a step (the two halves of the
    matrix instruction's A operand), every eighth of K, against scale * code +
    bias to a thousandth of a code step (float32 output: nothing is rounded)."""
    import mflux_amd
    from gpu_util import to_dev, u32_to_dev

    o = oracle
    K, N = 3072, 64
    w = o.f32_to_bf16_bits(seeded(65, 1, (N, K), 0.02))
    wq, s, b = o.c_quantize(w, o.BF16, 64, bits)
    exact = o.dequantize_exact(wq, s, b, o.BF16, 64, bits).astype(np.float64)
    step = np.abs(o.bf16_bits_to_f32(s).astype(np.float64))
    ks = list(range(0, 260)) + [383, 384, 385, 447, 448, 1023, 1024, 1535, 1536, 2687, 2688, 3008, 3071]
    for k0 in ks:
        cols = [(k0 + 389 * m) % K for m in range(M)]
        xf = np.zeros((M, K), dtype=np.float32)
        for m, k in enumerate(cols):
            xf[m, k] = 1.0
        y = mflux_amd.quantized_matmul(to_dev(o.f32_to_bf16_bits(xf), o.BF16).float(), u32_to_dev(wq),
                                       to_dev(s, o.BF16), to_dev(b, o.BF16), group_size=64, bits=bits)
        got = y.cpu().numpy().astype(np.float64)
        for m, k in enumerate(cols):
            assert np.all(np.abs(got[m] - exact[:, k]) <= 1e-3 * step[:, k // 64]), (k0, m)


def test_oct_unit_weight_is_exact(oracle):
    """Codes 1 on the diagonal and 0 elsewhere, scale 1, bias 0: y = x exactly
    (float32 output), although every code enters the matrix instruction as
    code - 128 -- the 128 * sum(xq) that this takes out is put back as an
    integer, before anything is rounded."""
    import mflux_amd
    from gpu_util import to_dev, u32_to_dev

    o = oracle
    K = N = 1024
    n = np.arange(N)
    wq = np.zeros((N, K // 4), dtype=np.uint32)
    wq[n, n // 4] = np.uint32(1) << (8 * (n % 4)).astype(np.uint32)
    one = o.f32_to_bf16_bits(np.ones((N, K // 64), np.float32))
    zero = o.f32_to_bf16_bits(np.zeros((N, K // 64), np.float32))
    x = o.f32_to_bf16_bits(np.abs(seeded(66, 0, (2, K), 1.0)) + np.float32(1.0))   # all positive: sum(xq) is large
    y = mflux_amd.quantized_matmul(to_dev(x, o.BF16).float(), u32_to_dev(wq), to_dev(one, o.BF16),
                                   to_dev(zero, o.BF16), group_size=64, bits=8)
    got = y.cpu().numpy().astype(np.float64)
    xf = o.bf16_bits_to_f32(x).astype(np.float64)
    # 15-bit fixed point of each eighth of a row: 2^-15 of the eighth's largest magnitude
    assert np.all(np.abs(got - xf) <= 2.0 ** -14 * np.abs(xf).max())
