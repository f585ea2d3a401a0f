"""GPU parity of mfq_layer_norm_modulate: LayerNorm without learned parameters
and the adaLN modulation, y = LayerNorm(x) * (1 + scale) + shift, as one pass.
Against float64 of the same formula (every element within 4 * 2^-8 of the row's
largest magnitude: the normalised value, 1 + scale, the product and the sum are
each rounded to bfloat16, half an ulp <= 2^-8 of the value each) and against the
reference's sequence of operations in torch, which rounds at the same points
(float32 sums in another order: a last place here and there)."""
import numpy as np
import pytest
import torch

from conftest import seeded

pytestmark = pytest.mark.gpu


def _ref64(x, scale, shift, eps, rows_per_vector):
    mean = x.mean(axis=-1, keepdims=True)
    var = ((x - mean) ** 2).mean(axis=-1, keepdims=True)
    y = (x - mean) / np.sqrt(var + eps)
    if scale is not None:
        idx = np.arange(x.shape[0]) // rows_per_vector
        y = y * (1.0 + scale[idx]) + shift[idx]
    return y


@pytest.mark.parametrize("M,K,B", [(1, 3072, 1), (5, 64, 1), (4608, 3072, 1), (1024, 1536, 2), (300, 3840, 3),
                                   (7, 8192, 1), (33, 200, 1), (64, 520, 4)])
@pytest.mark.parametrize("modulated", [True, False])
def test_layer_norm_modulate(oracle, M, K, B, modulated):
    import mflux_amd
    from gpu_util import to_dev

    o = oracle
    print(f"M={M} K={K} B={B} modulated={modulated}", flush=True)
    xh = o.f32_to_bf16_bits(seeded(61, 0, (M, K), 1.0) * np.float32(1.7) + np.float32(0.3))
    sch = o.f32_to_bf16_bits(seeded(61, 1, (B, K), 0.3))
    shh = o.f32_to_bf16_bits(seeded(61, 2, (B, K), 0.3))
    x = to_dev(xh, o.BF16).reshape(B, M // B, K) if M % B == 0 and B > 1 else to_dev(xh, o.BF16)
    if M % B:
        pytest.skip("rows do not divide into batch entries")
    sc, sh = (to_dev(sch, o.BF16), to_dev(shh, o.BF16)) if modulated else (None, None)
    guard = torch.full((4, K), 7.0, device="cuda", dtype=torch.bfloat16)
    y = mflux_amd.layer_norm_modulate(x, sc if B > 1 or sc is None else sc[0], sh if B > 1 or sh is None else sh[0], eps=1e-6)
    assert y.shape == x.shape and y.dtype == torch.bfloat16
    ref = _ref64(o.bf16_bits_to_f32(xh).astype(np.float64),
                 o.bf16_bits_to_f32(sch).astype(np.float64) if modulated else None,
                 o.bf16_bits_to_f32(shh).astype(np.float64) if modulated else None, 1e-6, M // B)
    got = y.reshape(M, K).double().cpu().numpy()
    err = np.abs(got - ref).max(axis=1) / np.abs(ref).max(axis=1)
    assert err.max() <= 4 * 2.0 ** -8, f"max |err| / ||row||inf = {err.max():.4g}"
    # the reference's own sequence of operations, in torch
    t = torch.nn.functional.layer_norm(x, (K,), eps=1e-6)
    if modulated:
        scb, shb = (sc[:, None, :], sh[:, None, :]) if B > 1 else (sc[0], sh[0])
        t = t * (1 + scb) + shb
    diff = (y.float() - t.float()).abs().reshape(M, K)
    # in last places of the larger of the result and 1: the product n * (1 + scale) is of order 1 and may all but
    # cancel against the shift, so a last place of the product is many of the sum's
    ulp = torch.maximum(y.float().abs(), t.float().abs()).reshape(M, K).clamp_min(1.0) * 2.0 ** -7
    assert float((diff / ulp).max()) <= 2.01
    assert float((diff > 0).float().mean()) < 0.05
    assert bool((guard == 7.0).all())


def test_layer_norm_modulate_f16_long_rows_and_validation(oracle):
    import mflux_amd
    from mflux_amd import _lib

    torch.manual_seed(8)
    x = torch.randn(20, 1024, device="cuda").to(torch.float16)
    sc = (torch.randn(1024, device="cuda") * 0.2).to(torch.float16)
    sh = (torch.randn(1024, device="cuda") * 0.2).to(torch.float16)
    y = mflux_amd.layer_norm_modulate(x, sc, sh)
    ref = _ref64(x.double().cpu().numpy(), sc.double().cpu().numpy()[None], sh.double().cpu().numpy()[None], 1e-6, 20)
    assert np.abs(y.double().cpu().numpy() - ref).max() <= 2.0 ** -8 * np.abs(ref).max()
    # rows beyond what the kernel holds in registers: the same operations composed
    xl = torch.randn(3, 8200, device="cuda").to(torch.bfloat16)
    yl = mflux_amd.layer_norm_modulate(xl)
    assert torch.equal(yl, torch.nn.functional.layer_norm(xl, (8200,), eps=1e-6))
    lib = _lib.load()
    y0 = torch.empty_like(xl)
    rc = lib.mfq_layer_norm_modulate(xl.data_ptr(), _lib.BF16, 3, 8200, None, None, 0, 1e-6, y0.data_ptr(), None)
    assert rc == _lib.MFQ_EUNSUPPORTED
    with pytest.raises(ValueError, match="come together"):
        mflux_amd.layer_norm_modulate(x, sc, None)
    # a flat row of equal values: variance 0, the normalised row is 0 and the result is the shift
    flat = torch.full((2, 1024), 3.0, device="cuda", dtype=torch.float16)
    assert torch.equal(mflux_amd.layer_norm_modulate(flat, sc, sh), sh.expand(2, 1024))
