"""GPU parity of the two-kernel large-M path (csrc/qmm_frag.hip): the scratch
copy of the weights is bit-identical to the oracle's dequantisation, laid out in
fragment order, and the product meets the matmul tolerance (1e-2 of the row's
largest reference magnitude) against the float64 oracle; the fused kernel, which
the same call falls back to without a workspace, agrees within the same bound.
"""
import numpy as np
import pytest
import torch

from conftest import seeded

pytestmark = pytest.mark.gpu

TOL = 1e-2


def _operands(o, cfg, M, K, N, bits, gs, dt, with_bias):
    def to_bits(a):
        return o._from_f32(a, dt)

    x = to_bits(seeded(cfg, 0, (M, K), 1.0))
    w = to_bits(seeded(cfg, 1, (N, K), 0.02))
    bias = to_bits(seeded(cfg, 2, (N,), 0.02)) if with_bias else None
    wq, s, b = o.c_quantize(w, dt, gs, bits)
    return x, wq, s, b, bias


def _to_f64(o, bits16, dt):
    return o._to_f32(bits16, dt).astype(np.float64)


def _call(lib, name, code, M, K, N, gs, bits, xd, wd, sd, bd, biasd, y, ws, ws_bytes):
    return getattr(lib, name)(xd.data_ptr(), code, M, K, wd.data_ptr(), sd.data_ptr(), bd.data_ptr(), code,
                              None if biasd is None else biasd.data_ptr(), N, gs, bits, y.data_ptr(), code,
                              None if ws is None else ws.data_ptr(), ws_bytes,
                              torch.cuda.current_stream().cuda_stream)


# 17 x 13 tiles = 221 of 256 CUs: the shape class the path takes; M and N ragged (N % 16 == 8)
# K = 512: four blocks of 64 k per wavefront and trip of the copy kernel; K = 384 and 640: two
# M = 2400: 10 x 17 tiles of 192 columns fit the 256 CUs, which is when the path uses those
@pytest.mark.parametrize("M", [4100, 2400])
@pytest.mark.parametrize("bits,gs,dtype,with_bias,K", [
    (4, 64, "bf16", True, 512), (8, 64, "bf16", False, 512), (4, 32, "bf16", False, 512), (8, 128, "bf16", True, 512),
    (4, 128, "f16", True, 512), (8, 32, "f16", False, 512), (4, 64, "bf16", False, 640), (8, 64, "f16", True, 384),
    # 3, 5 and 6 bits: the copy cut out of MLX's bit stream (32 codes to BITS words), then the same GEMM
    (3, 64, "bf16", True, 512), (5, 32, "bf16", False, 384), (6, 128, "f16", True, 512), (5, 64, "f16", False, 640),
    (3, 32, "f16", False, 384), (6, 64, "bf16", True, 640)])
def test_two_kernel_path_scratch_copy_and_product(oracle, bits, gs, dtype, with_bias, K, M):
    from gpu_util import to_dev, u32_to_dev
    from mflux_amd import _lib

    o = oracle
    lib = _lib.load()
    dt = o.BF16 if dtype == "bf16" else o.F16
    code = _lib.BF16 if dtype == "bf16" else _lib.F16
    N = 3208
    need = lib.mfq_qmm_t_workspace_bytes(M, K, N, gs, bits)
    n16 = (N + 15) // 16 * 16
    assert need == n16 * K * 2, "the shape must take the two-kernel path, uncut"
    x, wq, s, b, bias = _operands(o, 90 + bits + gs, M, K, N, bits, gs, dt, with_bias)
    xd, wd, sd, bd = to_dev(x, dt), u32_to_dev(wq), to_dev(s, dt), to_dev(b, dt)
    biasd = None if bias is None else to_dev(bias, dt)
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
    y = torch.empty(M, N, dtype=xd.dtype, device="cuda")
    assert _call(lib, "mfq_qmm_t_ws", code, M, K, N, gs, bits, xd, wd, sd, bd, biasd, y, ws, need) == 0
    torch.cuda.synchronize()

    # the scratch copy: blocks of 16 rows x 64 k as [half][q][c16][8], value (q, half, e) = k 16 q + 8 half + e
    copy = ws.view(torch.int16).view(n16 // 16, K // 64, 2, 4, 16, 8).permute(0, 4, 1, 3, 2, 5).reshape(n16, K)
    got = copy.cpu().numpy().view(np.uint16)
    w_hat = o.dequantize_exact(wq, s, b, dt, gs, bits).astype(np.float32)  # float32 fma of exact operands
    want = o._from_f32(w_hat, dt)
    assert np.array_equal(got[:N], want)
    assert np.array_equal(got[N:], np.broadcast_to(want[N - 1], (n16 - N, K)))  # rows past N repeat the last one

    ref = o.quantized_matmul_f64(_to_f64(o, x, dt), wq, s, b, dt, gs, bits,
                                 bias_f64=None if bias is None else _to_f64(o, bias, dt))
    row_inf = np.abs(ref).max(axis=-1, keepdims=True)
    err = np.abs(y.double().cpu().numpy() - ref) / row_inf
    assert err.max() <= TOL, err.max()

    # without a workspace the fused kernel (for 3, 5 and 6 bits: the 128-column-tile kernel) takes the call: same bound
    y_fused = torch.empty_like(y)
    assert _call(lib, "mfq_qmm_t_ws", code, M, K, N, gs, bits, xd, wd, sd, bd, biasd, y_fused, None, 0) == 0
    torch.cuda.synchronize()
    err_fused = np.abs(y_fused.double().cpu().numpy() - ref) / row_inf
    assert err_fused.max() <= TOL, err_fused.max()
    assert not torch.equal(y_fused, torch.zeros_like(y_fused))


# The untransposed product (the input gradient) on the same GEMM: the copy is the TRANSPOSE of the dequantised
# weight in fragment order.  10 x 13 tiles, the last column of tiles ragged; N (the reduction) of four, three and
# five pairs of 64
@pytest.mark.parametrize("bits,gs,dtype,N", [
    (4, 64, "bf16", 512), (8, 64, "bf16", 512), (4, 32, "f16", 384), (8, 128, "f16", 640), (4, 128, "bf16", 640),
    (8, 32, "bf16", 384)])
def test_two_kernel_path_untransposed_copy_and_product(oracle, bits, gs, dtype, N):
    from gpu_util import to_dev, u32_to_dev
    from mflux_amd import _lib

    o = oracle
    lib = _lib.load()
    dt = o.BF16 if dtype == "bf16" else o.F16
    code = _lib.BF16 if dtype == "bf16" else _lib.F16
    M, K = 2400, {32: 3232, 64: 3264, 128: 3200}[gs]     # whole groups: the output width is a multiple of 32
    k16 = (K + 15) // 16 * 16
    need = lib.mfq_qmm_n_workspace_bytes(M, N, K, gs, bits)
    assert need == k16 * N * 2, "the shape must take the two-kernel path, uncut"
    g = o._from_f32(seeded(120 + bits + gs, 0, (M, N), 1.0), dt)
    w = o._from_f32(seeded(120 + bits + gs, 1, (N, K), 0.02), dt)
    wq, s, b = o.c_quantize(w, dt, gs, bits)
    gd, wd, sd, bd = to_dev(g, dt), u32_to_dev(wq), to_dev(s, dt), to_dev(b, dt)
    stream = torch.cuda.current_stream().cuda_stream
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
    y = torch.empty(M, K, dtype=gd.dtype, device="cuda")
    print(f"bits={bits} gs={gs} {dtype} M={M} N={N} K={K}", flush=True)
    assert lib.mfq_qmm_n_ws(gd.data_ptr(), code, M, N, wd.data_ptr(), sd.data_ptr(), bd.data_ptr(), code, K, gs, bits,
                            y.data_ptr(), code, ws.data_ptr(), need, stream) == 0
    torch.cuda.synchronize()

    # blocks of 16 output columns k x 64 n as [half][q][c16][8], value (q, half, e) = n 16 q + 8 half + e
    copy = ws.view(torch.int16).view(k16 // 16, N // 64, 2, 4, 16, 8).permute(0, 4, 1, 3, 2, 5).reshape(k16, N)
    got = copy.cpu().numpy().view(np.uint16)
    w_hat = o.dequantize_exact(wq, s, b, dt, gs, bits)                     # [N, K] in float64, exact
    want = o._from_f32(w_hat.astype(np.float32), dt).T                      # [K, N]
    assert np.array_equal(got[:K], want)

    ref = _to_f64(o, g, dt) @ w_hat
    row_inf = np.abs(ref).max(axis=-1, keepdims=True)
    err = np.abs(y.double().cpu().numpy() - ref) / row_inf
    assert err.max() <= TOL, err.max()

    # the one-kernel form of the same call (no workspace): same bound
    y_one = torch.empty_like(y)
    assert lib.mfq_qmm_n(gd.data_ptr(), code, M, N, wd.data_ptr(), sd.data_ptr(), bd.data_ptr(), code, K, gs, bits,
                         y_one.data_ptr(), code, stream) == 0
    torch.cuda.synchronize()
    assert (np.abs(y_one.double().cpu().numpy() - ref) / row_inf).max() <= TOL


def test_two_kernel_path_untransposed_one_hot_and_k_cut(oracle):
    """One-hot rows of x pick rows of the dequantised weight, rounded once: bit
    for bit.  And a shape whose tile sequence has a tail, cut along the
    reduction into float32 planes (19 x 14 tiles = 266 on 256 compute units)."""
    import mflux_amd
    from gpu_util import raw, to_dev, u32_to_dev
    from mflux_amd import _lib

    o = oracle
    lib = _lib.load()
    for bits in (4, 8):
        M, N, K = 4700, 1024, 3520
        assert lib.mfq_qmm_n_workspace_bytes(M, N, K, 64, bits) > (K + 15) // 16 * 16 * N * 2 + 255, "planes too"
        w = o.f32_to_bf16_bits(seeded(130 + bits, 1, (N, K), 0.02))
        wq, s, b = o.c_quantize(w, o.BF16, 64, bits)
        hot = (np.arange(M) * 5 + 3) % N
        x = np.zeros((M, N), dtype=np.float32)
        x[np.arange(M), hot] = 1.0
        y = mflux_amd.quantized_matmul(to_dev(o.f32_to_bf16_bits(x), o.BF16), u32_to_dev(wq), to_dev(s, o.BF16),
                                       to_dev(b, o.BF16), transpose=False, group_size=64, bits=bits)
        expect = o.f32_to_bf16_bits(o.dequantize_exact(wq, s, b, o.BF16, 64, bits).astype(np.float32))[hot]
        assert np.array_equal(raw(y), expect)


def test_workspace_tells_the_path():
    """The workspace the library asks for tells which path a shape takes: the 16-bit
    copy (plus the planes of a K cut behind it) from 2048 activation rows on, the
    fused kernels' planes (or nothing) below."""
    from mflux_amd import _lib

    lib = _lib.load()
    if torch.cuda.get_device_properties(0).multi_processor_count != 256:
        pytest.skip("tile counts below are for 256 CUs")
    q = lib.mfq_qmm_t_workspace_bytes
    plane = 256 * 256 * 4
    assert q(4608, 3072, 21504, 64, 4) == 21504 * 3072 * 2      # FLUX single block, linear1: no cut
    assert q(4608, 15360, 3072, 64, 4) == 3072 * 15360 * 2      # linear2: 216 tiles, no cut
    assert q(4096, 3072, 3072, 64, 4) == 3072 * 3072 * 2        # 192 tiles: one short round, not worth cutting
    cut = q(6889, 3072, 3072, 64, 4) - 3072 * 3072 * 2          # one round + 68 tiles: the tail cut along K
    assert cut > 0 and cut % (68 * plane) == 0
    assert q(1024, 3072, 21504, 64, 4) % plane == 0             # four rows of tiles: the fused kernel (and its cut)
    assert q(4608, 3072, 21504, 64, 5) == 21504 * 3072 * 2      # 3, 5, 6 bits: the same copy, cut out of the bit stream,
    rest = q(1024, 3072, 21504, 64, 6) - 21504 * 3072 * 2       # from 1024 rows on (what it replaces there is slower);
    assert rest > 0 and rest % plane == 0                       # 336 tiles: one round + 80, the tail cut along K
    assert q(512, 3072, 21504, 64, 3) == 0                      # below: the 128-column-tile kernel, uncut here


@pytest.mark.parametrize("bits,dtype", [(4, "bf16"), (8, "f16")])
def test_two_kernel_path_with_a_k_cut(oracle, bits, dtype):
    """264 tiles on 256 CUs: the eight of the last round are cut along K into planes
    behind the copy; ragged M; bias; against the float64 oracle, and without the
    planes' part of the workspace (tiles then run whole) the same bound."""
    from gpu_util import to_dev, u32_to_dev
    from mflux_amd import _lib

    o = oracle
    lib = _lib.load()
    if torch.cuda.get_device_properties(0).multi_processor_count != 256:
        pytest.skip("tile counts below are for 256 CUs")
    dt = o.BF16 if dtype == "bf16" else o.F16
    code = _lib.BF16 if dtype == "bf16" else _lib.F16
    M, K, N = 2100, 2048, 7440  # 9 x 30 tiles = 270: 14 in the last round; N % 16 == 0, N % 256 != 0
    need = lib.mfq_qmm_t_workspace_bytes(M, K, N, 64, bits)
    copy = N * K * 2
    assert need == copy + 14 * 8 * 256 * 256 * 4
    x, wq, s, b, bias = _operands(o, 120 + bits, M, K, N, bits, 64, dt, True)
    xd, wd, sd, bd, biasd = to_dev(x, dt), u32_to_dev(wq), to_dev(s, dt), to_dev(b, dt), to_dev(bias, dt)
    ref = o.quantized_matmul_f64(_to_f64(o, x, dt), wq, s, b, dt, 64, bits, bias_f64=_to_f64(o, bias, dt))
    row_inf = np.abs(ref).max(axis=-1, keepdims=True)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    for ws_bytes in (need, copy):
        y = torch.full((M, N), float("nan"), dtype=xd.dtype, device="cuda")
        assert _call(lib, "mfq_qmm_t_ws", code, M, K, N, 64, bits, xd, wd, sd, bd, biasd, y, ws, ws_bytes) == 0
        torch.cuda.synchronize()
        err = np.abs(y.double().cpu().numpy() - ref) / row_inf
        assert err.max() <= TOL, (ws_bytes, err.max())


@pytest.mark.parametrize("bits,dtype,M,K,N", [(4, "bf16", 4608, 256, 7680), (8, "f16", 2100, 512, 7688)])
def test_two_kernel_path_deferred_stores(oracle, bits, dtype, M, K, N):
    """More tiles than CUs, run whole (the workspace holds the copy only): a tile without
    an output bias that lies inside y and has a successor on its workgroup is stored by
    that successor's first step.  A bias of -0.0 changes no bit of the result but takes
    every tile through the immediate epilogue, so the two calls must agree bit for bit;
    the float64 oracle bounds both.  The second shape has ragged edges in M and N (whose
    tiles are never deferred) next to deferred interior tiles."""
    from gpu_util import to_dev, u32_to_dev
    from mflux_amd import _lib

    o = oracle
    lib = _lib.load()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    assert ((M + 255) // 256) * ((N + 255) // 256) > cus + 16
    dt = o.BF16 if dtype == "bf16" else o.F16
    code = _lib.BF16 if dtype == "bf16" else _lib.F16
    x, wq, s, b, _ = _operands(o, 140 + bits, M, K, N, bits, 64, dt, False)
    xd, wd, sd, bd = to_dev(x, dt), u32_to_dev(wq), to_dev(s, dt), to_dev(b, dt)
    neg_zero = torch.full((N,), -0.0, dtype=xd.dtype, device="cuda")
    copy = (N + 15) // 16 * 16 * K * 2
    ws = torch.empty(copy, dtype=torch.uint8, device="cuda")
    ys = []
    for biasd in (None, neg_zero):
        y = torch.full((M, N), float("nan"), dtype=xd.dtype, device="cuda")
        assert _call(lib, "mfq_qmm_t_ws", code, M, K, N, 64, bits, xd, wd, sd, bd, biasd, y, ws, copy) == 0
        torch.cuda.synchronize()
        ys.append(y)
    assert torch.equal(ys[0].view(torch.int16), ys[1].view(torch.int16))
    ref = o.quantized_matmul_f64(_to_f64(o, x, dt), wq, s, b, dt, 64, bits)
    row_inf = np.abs(ref).max(axis=-1, keepdims=True)
    err = np.abs(ys[0].double().cpu().numpy() - ref) / row_inf
    assert err.max() <= TOL, err.max()
    # A real bias: deferred stores add it (an instantiation of its own).  The same two roundings as a
    # separate add on the 16-bit result, so y(bias) == round(y(no bias) + bias) bit for bit.
    bias = to_dev(o._from_f32(seeded(141 + bits, 2, (N,), 0.02), dt), dt)
    y = torch.full((M, N), float("nan"), dtype=xd.dtype, device="cuda")
    assert _call(lib, "mfq_qmm_t_ws", code, M, K, N, 64, bits, xd, wd, sd, bd, bias, y, ws, copy) == 0
    torch.cuda.synchronize()
    want = (ys[0].float() + bias.float()).to(xd.dtype)
    assert torch.equal(y.view(torch.int16), want.view(torch.int16))


def test_two_kernel_path_epilogues_and_graph_replay(oracle):
    """GELU from a column on, gate * y + residual and SwiGLU through the two-kernel
    path against the composed reference, and a captured call replayed bit for bit."""
    import mflux_amd
    from gpu_util import to_dev, u32_to_dev

    o = oracle
    M, K, N, bits = 4100, 512, 3200, 4
    x, wq, s, b, bias = _operands(o, 97, M, K, N, bits, 64, o.BF16, True)
    xd, wd, sd, bd, biasd = to_dev(x, o.BF16), u32_to_dev(wq), to_dev(s, o.BF16), to_dev(b, o.BF16), to_dev(bias, o.BF16)
    gate = to_dev(o.f32_to_bf16_bits(seeded(97, 3, (N,), 1.0)), o.BF16)
    res = to_dev(o.f32_to_bf16_bits(seeded(97, 4, (M, N), 1.0)), o.BF16)
    plain = mflux_amd.quantized_matmul(xd, wd, sd, bd, bits=bits, bias=biasd)

    def close(got, want, extra_roundings):
        bound = TOL + extra_roundings * 2.0 ** -8
        scale = want.double().abs().amax(dim=-1, keepdim=True).clamp_min(1e-30)
        err = ((got.double() - want.double()).abs() / scale).max().item()
        assert err <= bound, err

    y = mflux_amd.quantized_matmul_epilogue(xd, wd, sd, bd, epilogue="gelu", bits=bits, bias=biasd, act_from=1600)
    want = torch.cat([plain[:, :1600], mflux_amd.gelu_approx(plain[:, 1600:])], dim=-1)
    close(y, want, 1)
    y = mflux_amd.quantized_matmul_epilogue(xd, wd, sd, bd, epilogue="gate_residual", bits=bits, bias=biasd, gate=gate,
                                            residual=res)
    close(y, res + gate * plain, 2)
    y = mflux_amd.quantized_matmul_epilogue(xd, wd, sd, bd, epilogue="swiglu", bits=bits, bias=biasd)
    close(y, mflux_amd.core.swiglu_unstack(plain), 3)

    # graph capture: the workspace comes from torch's allocator inside the capture; every replay equals the eager result
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        mflux_amd.quantized_matmul(xd, wd, sd, bd, bits=bits, bias=biasd)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y_g = mflux_amd.quantized_matmul(xd, wd, sd, bd, bits=bits, bias=biasd)
    for _ in range(3):
        y_g.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_g, plain)
        mflux_amd.quantized_matmul(xd, wd, sd, bd, bits=bits)  # eager work between the replays
        torch.cuda.synchronize()


def test_two_kernel_path_is_reproducible_bit_for_bit():
    """The same call again and again gives the same bits -- whole tiles, a K cut, a
    LoRA update and an epilogue; with eager work of other shapes in between.  (The
    matrix instructions of this path are assembly the compiler's hazard checks do
    not see; a result read or overwritten in flight would show up here as a
    difference between runs.)"""
    import mflux_amd

    torch.manual_seed(11)
    dev = "cuda"
    cases = [(4608, 1024, 3072, 4, 0), (2100, 2048, 7440, 8, 0), (4608, 512, 3328, 4, 32), (4400, 3072, 21504, 4, 0)]
    for M, K, N, bits, rank in cases:
        x = torch.randn(M, K, device=dev, dtype=torch.bfloat16)
        w = (torch.randn(N, K, device=dev) * 0.02).to(torch.bfloat16)
        bias = torch.randn(N, device=dev, dtype=torch.bfloat16)
        wq, s, b = mflux_amd.quantize(w, 64, bits)
        low_rank = None
        if rank:
            low_rank = (torch.randn(M, rank, device=dev, dtype=torch.bfloat16),
                        (torch.randn(N, rank, device=dev) * 0.05).to(torch.bfloat16))
        other = torch.randn(300, K, device=dev, dtype=torch.bfloat16)

        def plain():
            return mflux_amd.quantized_matmul(x, wq, s, b, bits=bits, bias=bias, low_rank=low_rank)

        def gelu():
            return mflux_amd.quantized_matmul_epilogue(x, wq, s, b, epilogue="gelu", bits=bits, bias=bias)

        for fn in (plain,) if rank else (plain, gelu):
            first = fn()
            for i in range(12 if M * K * N < 1e11 else 4):
                mflux_amd.quantized_matmul(other, wq, s, b, bits=bits)  # another kernel in between
                again = fn()
                assert torch.equal(first, again), (M, K, N, bits, rank, fn.__name__, i)
        assert bool(torch.isfinite(first).all())


@pytest.mark.parametrize("bits,dtype,M,K,N,with_bias", [
    (4, "bf16", 4608, 256, 7680, False),   # 540 tiles: deferred stores, a K cut of the last 28
    (8, "f16", 2400, 512, 3208, True),     # 192-column tiles, ragged
    (4, "bf16", 300, 1024, 2304, True),    # few rows: the same kernel on tiles the other paths would not give it
])
def test_prepared_copy_gives_the_two_kernel_paths_bits(oracle, bits, dtype, M, K, N, with_bias):
    """mfq_qmm_t_prepare + mfq_qmm_t_prepared are the two kernels of a large
    mfq_qmm_t_ws call apart: the copy is the same bytes, the product the same
    bits (first two shapes, which mfq_qmm_t_ws runs on that path), and the
    float64 oracle bounds it for any M."""
    from gpu_util import to_dev, u32_to_dev
    from mflux_amd import _lib

    o = oracle
    lib = _lib.load()
    dt = o.BF16 if dtype == "bf16" else o.F16
    code = _lib.BF16 if dtype == "bf16" else _lib.F16
    x, wq, s, b, bias = _operands(o, 160 + bits, M, K, N, bits, 64, dt, with_bias)
    xd, wd, sd, bd = to_dev(x, dt), u32_to_dev(wq), to_dev(s, dt), to_dev(b, dt)
    biasd = None if bias is None else to_dev(bias, dt)
    stream = torch.cuda.current_stream().cuda_stream
    nbytes = lib.mfq_qmm_t_prepared_bytes(N, K, bits)
    assert nbytes == (N + 15) // 16 * 16 * K * 2
    copy = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    assert lib.mfq_qmm_t_prepare(wd.data_ptr(), sd.data_ptr(), bd.data_ptr(), code, N, K, 64, bits, copy.data_ptr(),
                                 stream) == 0
    ws_bytes = lib.mfq_qmm_t_prepared_workspace_bytes(M, K, N)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device="cuda")
    y = torch.full((M, N), float("nan"), dtype=xd.dtype, device="cuda")
    assert lib.mfq_qmm_t_prepared(xd.data_ptr(), code, M, K, copy.data_ptr(),
                                  None if biasd is None else biasd.data_ptr(), N, y.data_ptr(), ws.data_ptr(),
                                  ws_bytes, stream) == 0
    torch.cuda.synchronize()
    ref = o.quantized_matmul_f64(_to_f64(o, x, dt), wq, s, b, dt, 64, bits,
                                 bias_f64=None if bias is None else _to_f64(o, bias, dt))
    err = np.abs(y.double().cpu().numpy() - ref) / np.abs(ref).max(axis=-1, keepdims=True)
    assert err.max() <= TOL, err.max()
    need = lib.mfq_qmm_t_workspace_bytes(M, K, N, 64, bits)
    if need >= nbytes and M >= 2048:
        full = torch.empty(need, dtype=torch.uint8, device="cuda")
        y_ws = torch.empty_like(y)
        assert _call(lib, "mfq_qmm_t_ws", code, M, K, N, 64, bits, xd, wd, sd, bd, biasd, y_ws, full, need) == 0
        torch.cuda.synchronize()
        assert torch.equal(full[:nbytes], copy)
        assert torch.equal(y_ws.view(torch.int16), y.view(torch.int16))


def test_quantized_linear_prepare():
    """QuantizedLinear.prepare(): same bits as the layer gives without it from
    2048 rows on, the ordinary kernels below that, and a new copy after the
    layer's tensors have been written to."""
    import mflux_amd

    torch.manual_seed(5)
    lin = mflux_amd.nn.QuantizedLinear(512, 3072, bias=True, group_size=64, bits=4, device="cuda")
    lin.bias.normal_(0, 0.02)
    x = torch.randn(2, 2304, 512, device="cuda", dtype=torch.bfloat16)
    small = torch.randn(7, 512, device="cuda", dtype=torch.bfloat16)
    y0, s0 = lin(x), lin(small)
    assert lin.prepare()
    assert "_prepared" not in lin.state_dict()
    assert torch.equal(lin(x), y0) and torch.equal(lin(small), s0)
    w2, sc2, b2 = mflux_amd.quantize(torch.randn(3072, 512, device="cuda", dtype=torch.bfloat16) * 0.05, 64, 4)
    lin.weight.copy_(w2), lin.scales.copy_(sc2), lin.biases.copy_(b2)
    y1 = mflux_amd.quantized_matmul(x, w2, sc2, b2, bias=lin.bias)
    assert not torch.equal(y1, y0)
    assert torch.equal(lin(x), y1)
    # 3, 5 and 6 bits have the same copy (cut out of the bit stream); a width the copy is not built for has none
    odd = mflux_amd.nn.QuantizedLinear(512, 3072, bias=False, group_size=64, bits=6, device="cuda")
    y_odd = odd(x)
    assert odd.prepare() and torch.equal(odd(x), y_odd)
    narrow = mflux_amd.nn.QuantizedLinear(192, 3072, bias=False, group_size=64, bits=4, device="cuda")
    assert not narrow.prepare()
    # the copy knows what it was made from: another dtype or width is refused, not multiplied
    copy = mflux_amd.prepare_weights(lin.weight, lin.scales, lin.biases, 64, 4)
    assert (copy.dtype, copy.output_dims, copy.input_dims, copy.bits) == (torch.bfloat16, 3072, 512, 4)
    with pytest.raises(ValueError, match="holds torch.bfloat16"):
        mflux_amd.quantized_matmul_prepared(x.half(), copy)
    with pytest.raises(ValueError, match="belongs to a weight of 3072 x 512"):
        mflux_amd.quantized_matmul_prepared(x[..., :256].contiguous(), copy)
    with pytest.raises(ValueError, match="what prepare_weights returned"):
        mflux_amd.quantized_matmul_prepared(x, copy.data)
    assert torch.equal(mflux_amd.quantized_matmul_prepared(x, copy, bias=lin.bias), lin(x))
    # a tensor assigned afresh (not written into) is noticed too, whatever address it gets
    lin.prepare()
    lin.weight = w2.clone()
    assert not lin._prepared_is_current()
    assert torch.equal(lin(x), y1) and lin._prepared_is_current()
    # the walk over a model: every quantized linear that has such a copy, and what they hold together
    model = torch.nn.Sequential(mflux_amd.nn.QuantizedLinear(512, 1024, device="cuda"), torch.nn.GELU(),
                                mflux_amd.nn.QuantizedLinear(1024, 512, bits=8, device="cuda"), odd, narrow)
    assert mflux_amd.nn.prepare(model) == 2 * (1024 * 512 + 512 * 1024 + 3072 * 512)
    assert mflux_amd.nn.prepare(model, min_output_dims=1024) == 2 * (1024 * 512 + 3072 * 512)
