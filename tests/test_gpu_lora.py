"""GPU parity of the LoRA path: the quantized matmul with a low-rank update
(`t @ bs.T` accumulated with the product) and the LoRALinear / FusedLoRALinear
wrappers, against float64 arithmetic on the same operands.

Tolerance as for the plain product: max |y - y_ref| <= 1e-2 * max|y_ref row|.
"""
import numpy as np
import pytest
import torch

from conftest import seeded

pytestmark = pytest.mark.gpu

TOL = 1e-2


def _operands(o, cfg, M, K, N, bits, gs, R, with_bias=True, dtype=None):
    dtype = o.BF16 if dtype is None else dtype
    to_bits = o.f32_to_bf16_bits if dtype == o.BF16 else (lambda a: a.astype(np.float16).view(np.uint16))
    x = to_bits(seeded(cfg, 0, (M, K), 1.0))
    w = to_bits(seeded(cfg, 1, (N, K), 0.02))
    bias = to_bits(seeded(cfg, 2, (N,), 0.02)) if with_bias else None
    # the update is of the order of the product itself, so a wrong or missing term cannot hide
    t = to_bits(seeded(cfg, 3, (M, R), 1.0))
    bs = to_bits(seeded(cfg, 4, (N, R), 1.0 / np.sqrt(R)))
    wq, s, b = o.c_quantize(w, dtype, gs, bits)
    return x, wq, s, b, bias, t, bs


def _f64(o, raw, dtype):
    if dtype == o.BF16:
        return o.bf16_bits_to_f32(raw).astype(np.float64)
    return raw.view(np.float16).astype(np.float64)


def _ref(o, x, wq, s, b, bias, t, bs, bits, gs, dtype):
    bf = None if bias is None else _f64(o, bias, dtype)
    y = o.quantized_matmul_f64(_f64(o, x, dtype), wq, s, b, dtype, gs, bits, bias_f64=bf)
    return y + _f64(o, t, dtype) @ _f64(o, bs, dtype).T


def _run(o, x, wq, s, b, bias, t, bs, bits, gs, dtype):
    import mflux_amd
    from gpu_util import to_dev, u32_to_dev

    y = mflux_amd.quantized_matmul(
        to_dev(x, dtype), u32_to_dev(wq), to_dev(s, dtype), to_dev(b, dtype), transpose=True, group_size=gs,
        bits=bits, bias=None if bias is None else to_dev(bias, dtype), low_rank=(to_dev(t, dtype), to_dev(bs, dtype)))
    torch.cuda.synchronize()
    return y


def _assert_close(y, ref, tol=TOL):
    got = y.detach().to(torch.float64).cpu().numpy()
    assert got.shape == ref.shape
    err = np.abs(got - ref) / np.maximum(np.abs(ref).max(axis=-1, keepdims=True), 1e-30)
    worst = float(err.max())
    assert worst <= tol, f"max |err| / ||row||inf = {worst:.4g} > {tol}"


# M, K, N: the two-kernel path from 2048 rows on (update behind the k loop; 2200 x 7504
# at K = 2048 has its last round cut along K, ragged M and N; rank 48 fills half of
# its last chunk of 32), the fused 256 x 256-tile kernel below that (2000 x 5000),
# the 128-column-tile kernel, the matvec kernels, K an odd multiple of 32
@pytest.mark.parametrize("bits,gs", [(4, 64), (8, 64), (4, 32), (8, 128)])
@pytest.mark.parametrize("M,K,N,R", [
    (2200, 512, 2304, 16), (2200, 2048, 7504, 32), (4608, 1024, 3072, 48), (1000, 1024, 5000, 16),
    (2000, 1024, 5000, 16),
    (300, 2048, 520, 16), (512, 3072, 768, 64), (100, 512, 1000, 128),
    (1, 3072, 1024, 16), (4, 3072, 1032, 32), (16, 512, 264, 16), (9, 256, 77, 16),
])
def test_low_rank_update_vs_f64(oracle, bits, gs, M, K, N, R):
    o = oracle
    args = _operands(o, 50, M, K, N, bits, gs, R, with_bias=(N % 2 == 0))
    _assert_close(_run(o, *args, bits, gs, o.BF16), _ref(o, *args, bits, gs, o.BF16))


@pytest.mark.parametrize("bits", [4, 8])
def test_low_rank_update_with_deferred_tile_stores(oracle, bits):
    """540 tiles on 256 CUs without an output bias: every workgroup's first tile is
    stored by the first step of its second one, after the update's matrix
    instructions have added to it; the last 28 tiles are cut along K."""
    o = oracle
    args = _operands(o, 54, 4608, 256, 7680, bits, 64, 16, with_bias=False)
    _assert_close(_run(o, *args, bits, 64, o.BF16), _ref(o, *args, bits, 64, o.BF16))


def test_low_rank_update_k_odd_multiple_of_32(oracle):
    o = oracle
    args = _operands(o, 51, 300, 96, 200, 4, 32, 16)
    _assert_close(_run(o, *args, 4, 32, o.BF16), _ref(o, *args, 4, 32, o.BF16))


@pytest.mark.parametrize("M", [1, 40])
@pytest.mark.parametrize("bits", [3, 5, 6])
def test_low_rank_update_odd_bit_widths(oracle, bits, M):
    o = oracle
    args = _operands(o, 52, M, 1024, 520, bits, 64, 32)
    _assert_close(_run(o, *args, bits, 64, o.BF16), _ref(o, *args, bits, 64, o.BF16))


@pytest.mark.parametrize("M,K,N", [(2200, 512, 2304), (300, 1024, 520), (2, 1024, 512)])
def test_low_rank_update_f16_and_float32_output(oracle, M, K, N):
    import mflux_amd
    from gpu_util import to_dev, u32_to_dev

    o = oracle
    x, wq, s, b, bias, t, bs = args = _operands(o, 53, M, K, N, 4, 64, 16, dtype=o.F16)
    ref = _ref(o, *args, 4, 64, o.F16)
    _assert_close(_run(o, *args, 4, 64, o.F16), ref)
    # float32 activations against 16-bit scales: float32 result
    y = mflux_amd.quantized_matmul(
        to_dev(x, o.F16).float(), u32_to_dev(wq), to_dev(s, o.F16), to_dev(b, o.F16), group_size=64, bits=4,
        bias=to_dev(bias, o.F16), low_rank=(to_dev(t, o.F16), to_dev(bs, o.F16)))
    assert y.dtype == torch.float32
    _assert_close(y, ref, tol=2e-3)


def test_low_rank_update_is_exact_on_integers(oracle):
    """Integer-valued operands keep every partial sum exactly representable, so
    the fused update must reproduce the integer result bit for bit: pins the
    fragment layout of both update operands (any row / k mix-up changes it)."""
    import mflux_amd

    rng = np.random.default_rng(7)
    M, K, N, R = 600, 256, 2304, 32
    x = torch.from_numpy(rng.integers(-2, 3, (M, K)).astype(np.float32)).cuda().to(torch.bfloat16)
    codes = rng.integers(0, 16, (N, K)).astype(np.float32)
    codes[:, ::64] = 0
    codes[:, 1::64] = 15      # every group spans 0..15: scale 1 (or -1), codes = values
    w = torch.from_numpy(codes).cuda().to(torch.bfloat16)
    wq, s, b = mflux_amd.quantize(w, 64, 4)
    assert torch.equal(mflux_amd.dequantize(wq, s, b, 64, 4), w)
    t = torch.from_numpy(rng.integers(-3, 4, (M, R)).astype(np.float32)).cuda().to(torch.bfloat16)
    bs = torch.from_numpy(rng.integers(-3, 4, (N, R)).astype(np.float32)).cuda().to(torch.bfloat16)
    y = mflux_amd.quantized_matmul(x.float(), wq, s, b, group_size=64, bits=4, low_rank=(t, bs))
    ref = x.double() @ w.double().t() + t.double() @ bs.double().t()
    assert torch.equal(y.double(), ref)


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
@pytest.mark.parametrize("M,K,R", [
    (4608, 3072, 16),      # the single-block linear1 with one rank-16 adapter: six steps of 32 k per wavefront
    (100, 15360, 48),      # ragged rows, three fragments of columns, thirty steps per wavefront
    (17, 96, 80),          # fewer steps (3) than wavefronts (16); two column blocks (64 + 16)
    (1, 32, 16),           # one row, one step
    (333, 1056, 128),      # 33 steps: the wavefronts' shares are uneven (3, 3, ..., 0)
])
def test_down_projection_vs_f64(oracle, dtype, M, K, R):
    """t = x @ A through the C ABI (at = A^T, [R, K]): float32 sums of exact products, rounded once:
    within one rounding of the float64 value (2^-8 relative for bfloat16, 2^-11
    for float16, of the row's largest |t|, plus the float32 summation error)."""
    from gpu_util import raw, to_dev
    from mflux_amd import _lib

    o = oracle
    lib = _lib.load()
    dt = o.BF16 if dtype == "bf16" else o.F16
    code = _lib.BF16 if dtype == "bf16" else _lib.F16
    x = o._from_f32(seeded(140 + R, 0, (M, K), 1.0), dt)
    at = o._from_f32(seeded(140 + R, 1, (R, K), 1.0 / np.sqrt(K)), dt)
    # A = at^T in the order the kernel wants it: af[f, s, q, c, e] = A[32 s + 8 q + e, 16 f + c]
    f_, s_, q_, c_, e_ = np.indices((R // 16, K // 32, 4, 16, 8))
    af = np.ascontiguousarray(at.T[32 * s_ + 8 * q_ + e_, 16 * f_ + c_])
    xd, ad = to_dev(x, dt), to_dev(af.reshape(-1, 8), dt)
    guard = torch.full((M + 2, R), 7.0, device="cuda", dtype=xd.dtype)
    t = guard[1:M + 1]
    print(f"{dtype} M={M} K={K} R={R}", flush=True)
    assert lib.mfq_low_rank_down(xd.data_ptr(), ad.data_ptr(), code, M, K, R, t.data_ptr(),
                                 torch.cuda.current_stream().cuda_stream) == 0
    torch.cuda.synchronize()
    ref = o._to_f32(x, dt).astype(np.float64) @ o._to_f32(at, dt).astype(np.float64).T
    err = np.abs(t.double().cpu().numpy() - ref) / np.abs(ref).max(axis=1, keepdims=True)
    assert err.max() <= (2.0 ** -8 if dtype == "bf16" else 2.0 ** -11) * 1.05, err.max()
    assert bool((guard[0] == 7.0).all()) and bool((guard[M + 1] == 7.0).all())
    # one-hot rows pick columns of at, bit for bit
    hot = (np.arange(M) * 7 + 3) % K
    xh = np.zeros((M, K), dtype=np.float32)
    xh[np.arange(M), hot] = 1.0
    th = torch.empty(M, R, device="cuda", dtype=xd.dtype)
    assert lib.mfq_low_rank_down(to_dev(o._from_f32(xh, dt), dt).data_ptr(), ad.data_ptr(), code, M, K, R,
                                 th.data_ptr(), torch.cuda.current_stream().cuda_stream) == 0
    assert np.array_equal(raw(th), at[:, hot].T)


def test_low_rank_argument_checks():
    import mflux_amd

    x = torch.randn(4, 128, device="cuda").to(torch.bfloat16)
    w = (torch.randn(64, 128, device="cuda") * 0.02).to(torch.bfloat16)
    wq, s, b = mflux_amd.quantize(w, 64, 4)
    t = torch.zeros(4, 16, device="cuda", dtype=torch.bfloat16)
    bs = torch.zeros(64, 16, device="cuda", dtype=torch.bfloat16)
    mflux_amd.quantized_matmul(x, wq, s, b, low_rank=(t, bs))
    with pytest.raises(ValueError, match="multiple of 16"):
        mflux_amd.quantized_matmul(x, wq, s, b, low_rank=(t[:, :8], bs[:, :8]))
    with pytest.raises(ValueError, match="low_rank must be"):
        mflux_amd.quantized_matmul(x, wq, s, b, low_rank=(t[:3], bs))
    with pytest.raises(ValueError, match="low_rank must be"):
        mflux_amd.quantized_matmul(x, wq, s, b, low_rank=(t, bs[:32]))
    with pytest.raises(ValueError, match="transpose=True"):
        mflux_amd.quantized_matmul(x[:, :64], wq, s, b, transpose=False, low_rank=(t, bs))
    with pytest.raises(ValueError, match="not differentiable"):
        mflux_amd.quantized_matmul(x.clone().requires_grad_(), wq, s, b, low_rank=(t, bs))


# ---- the wrappers ----------------------------------------------------------------
def _layer_ref(x, w_deq, bias, loras):
    y = x.double() @ w_deq.double().t()
    if bias is not None:
        y = y + bias.double()
    for lora in loras:
        y = y + lora.scale * (x.double() @ lora.lora_A.double()) @ lora.lora_B.double()
    return y.detach().cpu().numpy()


@pytest.mark.parametrize("bits", [4, 8, 6])
@pytest.mark.parametrize("M", [1, 300, 2200])
def test_lora_linear_on_quantized_base(bits, M):
    """LoRALinear.from_linear(QuantizedLinear): the fused call (no_grad) and the
    composition of separate matmuls (gradients enabled) both match float64 on
    the dequantised weight."""
    import mflux_amd
    from mflux_amd.lora import LoRALinear

    torch.manual_seed(3)
    K, N = 1024, 2304
    lin = torch.nn.Linear(K, N, bias=True, device="cuda", dtype=torch.bfloat16)
    q = mflux_amd.nn.QuantizedLinear.from_linear(lin, 64, bits)
    lora = LoRALinear.from_linear(q, r=16, scale=0.75)
    assert lora.linear is q and lora.lora_A.shape == (K, 16) and lora.lora_B.shape == (16, N)
    with torch.no_grad():
        lora.lora_B.mul_(8.0)   # an update comparable to the base output
    x = torch.randn(M, K, device="cuda").to(torch.bfloat16)
    ref = _layer_ref(x, mflux_amd.dequantize(q.weight, q.scales, q.biases, 64, bits), q.bias, [lora])
    with torch.no_grad():
        y = lora(x)
    assert y.dtype == torch.bfloat16 and not y.requires_grad
    _assert_close(y, ref)
    y_grad = lora(x)     # gradients enabled: the reference's composition, differentiable in A and B
    assert y_grad.requires_grad
    _assert_close(y_grad, ref, tol=2e-2)   # every intermediate rounded to bfloat16
    y_grad.float().sum().backward()
    assert lora.lora_A.grad is not None and lora.lora_B.grad is not None


def test_fused_lora_linear_several_adapters():
    """FusedLoRALinear with adapters of ranks 8, 16 and 4 (28 -> padded to 32);
    changing a scale or a tensor is seen by the next call."""
    import mflux_amd
    from mflux_amd.lora import FusedLoRALinear, LoRALinear

    torch.manual_seed(4)
    K, N, M = 512, 2304, 2200
    lin = torch.nn.Linear(K, N, bias=True, device="cuda", dtype=torch.bfloat16)
    q = mflux_amd.nn.QuantizedLinear.from_linear(lin, 64, 4)
    loras = [LoRALinear.from_linear(q, r=r, scale=sc) for r, sc in ((8, 1.0), (16, -0.5), (4, 2.0))]
    with torch.no_grad():
        for lora in loras:
            lora.lora_B.mul_(6.0)
    fused = FusedLoRALinear(q, loras)
    x = torch.randn(M, K, device="cuda").to(torch.bfloat16)
    w_deq = mflux_amd.dequantize(q.weight, q.scales, q.biases, 64, 4)
    with torch.no_grad():
        _assert_close(fused(x), _layer_ref(x, w_deq, q.bias, loras))
        loras[1].scale = 1.5
        _assert_close(fused(x), _layer_ref(x, w_deq, q.bias, loras))
        loras[2].lora_B.mul_(-1.0)
        _assert_close(fused(x), _layer_ref(x, w_deq, q.bias, loras))
        # leading batch dimension, as the transformer blocks pass it
        _assert_close(fused(x[None]), _layer_ref(x, w_deq, q.bias, loras)[None])


def test_lora_linear_on_plain_linear():
    from mflux_amd.lora import LoRALinear

    torch.manual_seed(5)
    lin = torch.nn.Linear(256, 128, bias=False, device="cuda", dtype=torch.bfloat16)
    lora = LoRALinear.from_linear(lin, r=8, scale=1.0)
    x = torch.randn(10, 256, device="cuda").to(torch.bfloat16)
    with torch.no_grad():
        _assert_close(lora(x), _layer_ref(x, lin.weight, None, [lora]), tol=2e-2)


@pytest.mark.parametrize("bits", [4, 8])
def test_bake_with_requantize_folds_the_adapters_into_the_codes(bits):
    """requantize=True: the base's codes become quantize(dequantize(W) + delta);
    the baked layer then answers like the wrapped one up to one requantization
    (a quantization step of the weight, not the matmul tolerance)."""
    import mflux_amd
    from mflux_amd.lora import FusedLoRALinear, LoRALinear, bake_and_strip_lora

    torch.manual_seed(6)
    K, N, M = 512, 768, 300
    lin = torch.nn.Linear(K, N, bias=True, device="cuda", dtype=torch.bfloat16)
    q = mflux_amd.nn.QuantizedLinear.from_linear(lin, 64, bits)
    loras = [LoRALinear.from_linear(q, r=8, scale=1.0), LoRALinear.from_linear(q, r=16, scale=-0.5)]
    holder = torch.nn.Sequential(FusedLoRALinear(q, loras))
    x = torch.randn(M, K, device="cuda").to(torch.bfloat16)
    w_old = mflux_amd.dequantize(q.weight, q.scales, q.biases, 64, bits)
    delta = sum(l.scale * (l.lora_A.float() @ l.lora_B.float()).t() for l in loras)
    target = (w_old.float() + delta).to(torch.bfloat16)
    with torch.no_grad():
        wrapped = holder(x).double()
    bake_and_strip_lora(holder, requantize=True)
    assert holder[0] is q
    wq, s, b = mflux_amd.quantize(target, 64, bits)
    assert torch.equal(q.weight, wq) and torch.equal(q.scales, s) and torch.equal(q.biases, b)
    w_new = mflux_amd.dequantize(q.weight, q.scales, q.biases, 64, bits).float()
    step = q.scales.float().abs().repeat_interleave(64, dim=1)
    # within one quantization step (the quantizer's own guarantee: it re-fits the scale to the group's
    # edge, so the far end can be off by more than half a step), plus the rounding of the stored scale
    # (times the code, up to 2^bits - 1) and of the dequantised value to bfloat16
    slack = 1.0 + (2 ** bits - 1) * 2.0 ** -8
    assert torch.all((w_new - target.float()).abs() <= slack * step + 2.0 ** -8 * target.float().abs() + 1e-6)
    with torch.no_grad():
        baked = q(x).double()
    err = (baked - wrapped).abs().max() / wrapped.abs().max()
    assert err < (0.15 if bits == 4 else 0.02)
