"""mfq_qmm_t_static, the entry point that allocates nothing: its float32 planes
live in a buffer inside the library's device image.  Called through the C ABI
and compared bit for bit with mfq_qmm_t_ws given a caller's workspace (the same
kernels on the same planes), on two calls in a row, the second smaller, so that
what the first call left in the shared buffer would show."""
import numpy as np
import pytest
import torch

from conftest import seeded

pytestmark = pytest.mark.gpu

STATIC_BYTES = 32 << 20  # MFQ_STATIC_SCRATCH_BYTES of include/mfq.h


def _operands(o, cfg, M, K, N, bits):
    from gpu_util import to_dev, u32_to_dev

    x = o.f32_to_bf16_bits(seeded(cfg, 0, (M, K), 1.0))
    w = o.f32_to_bf16_bits(seeded(cfg, 1, (N, K), 0.02))
    bias = o.f32_to_bf16_bits(seeded(cfg, 2, (N,), 0.02))
    wq, s, b = o.c_quantize(w, o.BF16, 64, bits)
    host = (x, wq, s, b, bias)
    dev = (to_dev(x, o.BF16), u32_to_dev(wq), to_dev(s, o.BF16), to_dev(b, o.BF16), to_dev(bias, o.BF16))
    return host, dev


def _call(lib, name, dev, M, K, N, bits, y, *extra):
    from mflux_amd import _lib

    x, wq, s, b, bias = dev
    stream = torch.cuda.current_stream().cuda_stream
    return getattr(lib, name)(x.data_ptr(), _lib.BF16, M, K, wq.data_ptr(), s.data_ptr(), b.data_ptr(), _lib.BF16,
                              bias.data_ptr(), N, 64, bits, y.data_ptr(), _lib.BF16, *extra, stream)


def test_static_scratch_matches_workspace_call_twice(oracle):
    from mflux_amd import _lib

    o = oracle
    lib = _lib.load()
    # (M, K, N, bits): a text-stream shape the 128-column kernel cuts along K, then a smaller one that is cut too;
    # the third call has 256 x 256 tiles whose short last round is cut (the fused large-M kernel's planes); the
    # fourth runs the two-kernel path with its 16-bit copy of the weights in the buffer, the fifth too, on
    # 192-column tiles (ragged in M and N)
    shapes = [(512, 3072, 3072, 4), (300, 2048, 1024, 8), (2040, 3072, 8448, 4), (4608, 512, 3072, 4),
              (2400, 512, 3208, 8)]
    for idx, (M, K, N, bits) in enumerate(shapes):
        need = lib.mfq_qmm_t_workspace_bytes(M, K, N, 64, bits)
        assert 0 < need <= STATIC_BYTES, f"case {idx} must exercise the scratch buffer (needs {need} bytes)"
        host, dev = _operands(o, 70 + idx, M, K, N, bits)
        print(f"static scratch case {idx}: M={M} K={K} N={N} bits={bits} planes={need} bytes", flush=True)
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        y_ws = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
        y_st = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
        rc = _call(lib, "mfq_qmm_t_ws", dev, M, K, N, bits, y_ws, ws.data_ptr(), need)
        assert rc == 0, lib.mfq_strerror(rc)
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        rc = _call(lib, "mfq_qmm_t_static", dev, M, K, N, bits, y_st)
        assert rc == 0, lib.mfq_strerror(rc)
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert torch.equal(y_st.view(torch.int16), y_ws.view(torch.int16)), f"case {idx}: results differ"
        # and both are the product: float64 on the same operands, tolerance 1e-2 of the row's largest magnitude
        x, wq, s, b, bias = host
        rows = np.linspace(0, M - 1, 16).astype(np.int64)
        ref = o.quantized_matmul_f64(o.bf16_bits_to_f32(x[rows]).astype(np.float64), wq, s, b, o.BF16, 64, bits,
                                     bias_f64=o.bf16_bits_to_f32(bias).astype(np.float64))
        got = y_st[torch.from_numpy(rows).cuda()].double().cpu().numpy()
        err = np.abs(got - ref).max(axis=1) / np.abs(ref).max(axis=1)
        assert err.max() <= 1e-2, f"case {idx}: {err.max()}"


def test_static_scratch_without_a_split_and_beyond_the_buffer(oracle):
    from mflux_amd import _lib

    o = oracle
    lib = _lib.load()
    # a shape that is not cut: the call is mfq_qmm_t
    M, K, N, bits = 5, 512, 384, 4
    assert lib.mfq_qmm_t_workspace_bytes(M, K, N, 64, bits) == 0
    _, dev = _operands(o, 75, M, K, N, bits)
    y_a = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    y_b = torch.empty_like(y_a)
    assert _call(lib, "mfq_qmm_t", dev, M, K, N, bits, y_a) == 0
    assert _call(lib, "mfq_qmm_t_static", dev, M, K, N, bits, y_b) == 0
    torch.cuda.synchronize()
    assert torch.equal(y_a.view(torch.int16), y_b.view(torch.int16))
    # a split that needs more planes than the buffer holds is refused before anything is launched
    M, K, N = 6889, 3072, 3072
    need = lib.mfq_qmm_t_workspace_bytes(M, K, N, 64, 4)
    if need <= STATIC_BYTES:
        pytest.skip(f"this device cuts M={M} into {need} bytes of planes, which fit")
    x = torch.zeros((M, K), dtype=torch.bfloat16, device="cuda")
    wq = torch.zeros((N, K // 8), dtype=torch.int32, device="cuda")
    s = torch.ones((N, K // 64), dtype=torch.bfloat16, device="cuda")
    y = torch.full((M, N), 7.0, dtype=torch.bfloat16, device="cuda")
    rc = _call(lib, "mfq_qmm_t_static", (x, wq, s, s, torch.zeros(N, dtype=torch.bfloat16, device="cuda")), M, K, N, 4, y)
    torch.cuda.synchronize()
    assert rc == _lib.MFQ_ESCRATCH
    assert b"scratch" in lib.mfq_strerror(rc)
    assert bool((y == 7.0).all()), "a refused call must not touch y"
