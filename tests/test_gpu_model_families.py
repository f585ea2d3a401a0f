"""GPU parity on the linears of the model families beside the benchmark's three:
FLUX.2 (hidden 6144, fused qkv+MLP projection, 24576-long rows into to_out, a
modulation matvec whose rows are longer than the eight-rows kernels take), the
Qwen2.5-VL and Qwen3 text encoders (hidden 3584 / 2560, grouped-query k/v
projections with few output features, 18944- and 9728-long MLP rows), ERNIE's
text encoder and SigLIP's MLP (K = 1152, N = 4304).  Each shape is cited to the
reference file that defines the layer; M is what the model feeds it (one row for
modulation and decoding, a prompt's or an image's tokens otherwise).

Checks per linear, as for the benchmark configurations: the packed weight against
the oracle's quantizer (bit for bit, a band of rows), sampled output rows against
the float64 product on the MLX-format operands (1e-2 of the row's largest
magnitude), every element against a dense bfloat16 product on the dequantized
weight (twice that: the dense product rounds the weights a second time).
"""
import numpy as np
import pytest
import torch

from conftest import seeded

pytestmark = pytest.mark.gpu

TOL = 1e-2

# (id, M, K, N, bits, group size, bias); the reference file that defines the layer
LINEARS = [
    # src/mflux/models/flux2/model/flux2_transformer/modulation.py:9 (dim -> 3 or 6 dim, one row of silu(temb))
    ("flux2_modulation_w8_m1", 1, 6144, 18432, 8, 64, False),
    ("flux2_modulation_w4_m1", 1, 6144, 36864, 4, 64, False),
    # src/mflux/models/flux2/model/flux2_transformer/parallel_self_attention.py:17,21
    ("flux2_qkv_mlp_proj", 2304, 6144, 55296, 4, 64, False),
    ("flux2_to_out_24576", 2304, 24576, 6144, 4, 64, False),
    # src/mflux/models/flux2/model/flux2_transformer/transformer.py:46 (context_embedder, 512 prompt tokens)
    ("flux2_context_embedder", 512, 7680, 6144, 8, 64, False),
    # src/mflux/models/qwen/model/qwen_text_encoder/qwen_mlp.py:8-10, qwen_attention.py:26-29
    ("qwen25vl_gate_proj", 320, 3584, 18944, 4, 64, False),
    ("qwen25vl_down_proj", 320, 18944, 3584, 4, 64, False),
    ("qwen25vl_q_proj", 320, 3584, 3584, 8, 64, True),
    ("qwen25vl_kv_proj", 320, 3584, 512, 8, 64, True),
    ("qwen25vl_gate_proj_m1", 1, 3584, 18944, 4, 64, False),
    ("qwen25vl_down_proj_m1", 1, 18944, 3584, 8, 64, False),
    ("qwen25vl_down_proj_m3", 3, 18944, 3584, 4, 64, False),
    # src/mflux/models/z_image/model/z_image_text_encoder/mlp.py:8-10, attention.py:21-24 (Qwen3-4B)
    ("qwen3_gate_proj", 300, 2560, 9728, 4, 64, False),
    ("qwen3_down_proj", 300, 9728, 2560, 4, 64, False),
    ("qwen3_q_proj_w6", 300, 2560, 4096, 6, 64, False),
    ("qwen3_kv_proj_w3", 300, 2560, 1024, 3, 64, False),
    ("qwen3_gate_proj_g32_m2", 2, 2560, 9728, 8, 32, False),
    # src/mflux/models/ernie_image/model/ernie_text_encoder/text_encoder.py:19-21
    ("ernie_text_gate_proj", 77, 4096, 12288, 4, 64, False),
    ("ernie_text_down_proj_w5", 77, 12288, 4096, 5, 64, False),
    # src/mflux/models/flux/model/siglip_vision_transformer/siglip_mlp.py:8 (27 x 27 patches)
    ("siglip_fc1", 729, 1152, 4304, 8, 64, True),
    # src/mflux/models/flux/model/redux_encoder/redux_encoder.py:8
    ("redux_up", 729, 1152, 12288, 4, 128, True),
]


@pytest.mark.parametrize("case", LINEARS, ids=[c[0] for c in LINEARS])
def test_model_family_linear(oracle, case):
    import mflux_amd
    from gpu_util import raw, to_dev

    o = oracle
    name, M, K, N, bits, gs, with_bias = case
    print(f"{name}: M={M} K={K} N={N} bits={bits} gs={gs} bias={with_bias}", flush=True)
    cfg = 60 + LINEARS.index(case)
    x = o.f32_to_bf16_bits(seeded(cfg, 0, (M, K), 1.0))
    w = o.f32_to_bf16_bits(seeded(cfg, 1, (N, K), 0.02))
    bias = o.f32_to_bf16_bits(seeded(cfg, 2, (N,), 0.02)) if with_bias else None
    xd, wd = to_dev(x, o.BF16), to_dev(w, o.BF16)
    biasd = None if bias is None else to_dev(bias, o.BF16)
    wq, s, b = mflux_amd.quantize(wd, gs, bits)
    band = slice(N // 2 - 24, N // 2 + 24)
    e_wq, e_s, e_b = o.c_quantize(w[band], o.BF16, gs, bits)
    assert np.array_equal(raw(wq[band]), e_wq) and np.array_equal(raw(s[band]), e_s) and np.array_equal(raw(b[band]), e_b)
    del wd, w
    guard = torch.full((8, N), 7.0, device="cuda", dtype=torch.bfloat16)
    y = mflux_amd.quantized_matmul(xd, wq, s, b, group_size=gs, bits=bits, bias=biasd)
    assert y.shape == (M, N) and y.dtype == torch.bfloat16
    rows = np.unique(np.clip(np.array([0, 1, 255, 256, M // 2, M - 257, M - 2, M - 1]), 0, M - 1))
    # the float64 product over a band of output features (all of them where the weight is small)
    cols = slice(0, N) if N * K <= 40_000_000 else slice(N // 3, N // 3 + 40_000_000 // K)
    ref = o.quantized_matmul_f64(o.bf16_bits_to_f32(x[rows]).astype(np.float64), raw(wq[cols]), raw(s[cols]),
                                 raw(b[cols]), o.BF16, gs, bits,
                                 bias_f64=None if bias is None else o.bf16_bits_to_f32(bias[cols]).astype(np.float64))
    dense = torch.matmul(xd, mflux_amd.dequantize(wq, s, b, gs, bits).t()).float()
    if biasd is not None:
        dense += biasd.float()
    row_inf = dense.abs().amax(dim=1, keepdim=True)
    got = y[torch.from_numpy(rows).cuda()][:, cols].double().cpu().numpy()
    scale = row_inf[torch.from_numpy(rows).cuda()].double().cpu().numpy()
    err = np.abs(got - ref).max(axis=1, keepdims=True) / scale
    assert err.max() <= TOL, f"{name}: max |err| / ||row||inf = {err.max():.4g}"
    assert float(((y.float() - dense).abs() / row_inf).max()) <= 2 * TOL
    assert bool((guard == 7.0).all())
