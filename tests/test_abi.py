"""The C ABI library loads without a GPU, exports every symbol its header
declares, and rejects bad arguments with an error code before touching the
device."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mfq.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mfq_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    for must in ("mfq_version", "mfq_strerror", "mfq_quantize_affine", "mfq_dequantize_affine", "mfq_dequantize_rows",
                 "mfq_qmm_t", "mfq_qmm_t_ws", "mfq_qmm_t_workspace_bytes", "mfq_qmm_t_low_rank", "mfq_low_rank_add", "mfq_low_rank_down",
                 "mfq_qmm_t_prepare", "mfq_qmm_t_prepared", "mfq_qmm_t_prepared_bytes", "mfq_qmm_t_prepared_workspace_bytes",
                 "mfq_qmv_silu"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from mflux_amd import _lib

    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} is declared in include/mfq.h but not exported"
    # and the binding knows a signature for each of them
    assert sorted(_lib.SIGNATURES) == declared_functions()


def test_status_strings():
    from mflux_amd import _lib

    lib = _lib.load()
    assert lib.mfq_version() >= 100
    assert lib.mfq_strerror(0) == b"ok"
    seen = set()
    for code in range(-8, 0):
        msg = lib.mfq_strerror(code)
        assert msg and msg != b"unknown status"
        seen.add(msg)
    assert len(seen) == 8
    assert lib.mfq_strerror(-99) == b"unknown status"


def test_argument_validation_needs_no_device():
    """Every check runs before the first HIP call, so a caller's mistake is an
    error code, never a launch."""
    from mflux_amd import _lib

    lib = _lib.load()
    E = {"dtype": -1, "group": -2, "bits": -3, "shape": -4, "null": -5, "align": -6, "unsupported": -8}
    buf = ctypes.create_string_buffer(4096 + 64)
    base = (ctypes.addressof(buf) + 15) & ~15
    q = lib.mfq_quantize_affine
    assert q(base, _lib.BF16, 4, 64, 48, 4, base, base, base, None) == E["group"]
    assert q(base, _lib.BF16, 4, 64, 64, 7, base, base, base, None) == E["bits"]
    assert q(base, 7, 4, 64, 64, 4, base, base, base, None) == E["dtype"]
    assert q(base, _lib.BF16, 4, 96, 64, 4, base, base, base, None) == E["shape"]
    assert q(base, _lib.BF16, 0, 64, 64, 4, base, base, base, None) == E["shape"]
    assert q(None, _lib.BF16, 4, 64, 64, 4, base, base, base, None) == E["null"]
    assert q(base + 2, _lib.BF16, 4, 64, 64, 4, base, base, base, None) == E["align"]
    d = lib.mfq_dequantize_affine
    assert d(base, base, base, _lib.BF16, 4, 64, 64, 2, base, _lib.BF16, None) == E["bits"]
    assert d(base, base, None, _lib.BF16, 4, 64, 64, 4, base, _lib.BF16, None) == E["null"]
    g = lib.mfq_dequantize_rows
    assert g(base, base, base, _lib.BF16, None, 2, 10, 128, 64, 4, base, _lib.BF16, None) == E["null"]
    assert g(base, base, base, _lib.BF16, base, 0, 10, 128, 64, 4, base, _lib.BF16, None) == E["shape"]
    assert g(base, base, base, _lib.BF16, base, 2, 10, 100, 64, 4, base, _lib.BF16, None) == E["shape"]
    assert g(base, base, base, _lib.BF16, base, 2, 10, 128, 64, 7, base, _lib.BF16, None) == E["bits"]
    m = lib.mfq_qmm_t
    args = dict(x=base, xd=_lib.BF16, M=4, K=128, wq=base, s=base, b=base, sd=_lib.BF16, bias=None, N=8, gs=64,
                bits=4, y=base, yd=_lib.BF16, stream=None)

    def call(**kw):
        a = {**args, **kw}
        return m(a["x"], a["xd"], a["M"], a["K"], a["wq"], a["s"], a["b"], a["sd"], a["bias"], a["N"], a["gs"],
                 a["bits"], a["y"], a["yd"], a["stream"])

    assert call(xd=_lib.F32) == E["dtype"]          # activations must be 16-bit
    assert call(sd=_lib.F16) == E["dtype"]          # and of the scales' type
    assert call(yd=_lib.F16) == E["dtype"]          # output: the scales' type or float32
    assert call(K=100) == E["shape"]
    assert call(M=0) == E["shape"]
    assert call(N=1 << 40) == E["shape"]
    assert call(wq=None) == E["null"]
    assert call(x=base + 4) == E["align"]
    assert call(gs=16) == E["group"]
    assert call(bits=5, y=base + 2) == E["align"]    # 3, 5, 6 bits, several rows: the GEMM writes y in 16-byte pieces
    assert call(bits=5, M=1, K=100) == E["shape"]    # the odd widths validate their arguments like the others
    n = lib.mfq_qmm_n                                 # the untransposed product: x [M, N], y [M, K]

    def call_n(x=base, xd=_lib.BF16, M=4, N=8, wq=base, s=base, b=base, sd=_lib.BF16, K=128, gs=64, bits=4, y=base,
               yd=_lib.BF16):
        return n(x, xd, M, N, wq, s, b, sd, K, gs, bits, y, yd, None)

    assert call_n(xd=_lib.F32) == E["dtype"]
    assert call_n(yd=_lib.F16) == E["dtype"]
    assert call_n(K=100) == E["shape"]
    assert call_n(N=0) == E["shape"]
    assert call_n(s=None) == E["null"]
    assert call_n(y=base + 8) == E["align"]
    assert call_n(bits=7) == E["bits"]
    assert call_n(N=12) == E["unsupported"]          # x rows are read in 16-byte pieces
    nws = lib.mfq_qmm_n_ws                            # the same checks in front of the workspace form
    assert nws(base, _lib.BF16, 4, 8, base, base, base, _lib.BF16, 100, 64, 4, base, _lib.BF16, None, 0, None) == E["shape"]
    assert nws(base, _lib.F32, 4, 8, base, base, base, _lib.BF16, 128, 64, 4, base, _lib.BF16, None, 0, None) == E["dtype"]
    nbytes = lib.mfq_qmm_n_workspace_bytes
    assert nbytes(4608, 21504, 3072, 64, 4) >= 3072 * 21504 * 2    # the transposed 16-bit copy (and planes)
    assert nbytes(4608, 21504, 3072, 64, 8) >= 3072 * 21504 * 2
    assert nbytes(4608, 21504, 3072, 64, 5) == 0      # 3, 5 and 6 bits: the one-kernel form only
    assert nbytes(512, 21504, 3072, 64, 4) == 0       # few rows of x: the one-kernel form
    assert nbytes(4608, 200, 3072, 64, 4) == 0        # the reduction is not whole pairs of 64
    assert nbytes(4608, 21504, 3000, 64, 4) == 0      # an error of the call itself: no workspace

    # the LoRA entry points: the rank comes in steps of 16 with both matrices present and aligned
    lr = lib.mfq_qmm_t_low_rank

    def call_lr(t=base, bs=base, rank=16, **kw):
        a = {**args, **kw}
        return lr(a["x"], a["xd"], a["M"], a["K"], a["wq"], a["s"], a["b"], a["sd"], a["bias"], a["N"], a["gs"],
                  a["bits"], t, bs, rank, a["y"], a["yd"], None, 0, a["stream"])

    assert call_lr(rank=8) == E["shape"]
    assert call_lr(rank=-16) == E["shape"]
    assert call_lr(rank=2048) == E["shape"]
    assert call_lr(t=None) == E["null"]
    assert call_lr(bs=base + 2) == E["align"]
    assert call_lr(K=100) == E["shape"]
    assert call_lr(rank=0, t=None, bs=None, wq=None) == E["null"]   # rank 0: the plain call's checks
    add = lib.mfq_low_rank_add
    assert add(base, base, _lib.F32, 4, 8, 16, base, _lib.F32, None) == E["dtype"]
    assert add(base, base, _lib.BF16, 4, 8, 16, base, _lib.F16, None) == E["dtype"]
    assert add(base, base, _lib.BF16, 0, 8, 16, base, _lib.BF16, None) == E["shape"]
    assert add(base, base, _lib.BF16, 4, 8, 24, base, _lib.BF16, None) == E["shape"]
    assert add(base, None, _lib.BF16, 4, 8, 16, base, _lib.BF16, None) == E["null"]
    assert add(base + 8, base, _lib.BF16, 4, 8, 16, base, _lib.BF16, None) == E["align"]
    down = lib.mfq_low_rank_down                      # t [M, rank] = x [M, K] @ at [rank, K]^T
    assert down(base, base, _lib.F32, 4, 64, 16, base, None) == E["dtype"]
    assert down(base, base, _lib.BF16, 4, 48, 16, base, None) == E["shape"]     # K in steps of 32
    assert down(base, base, _lib.BF16, 4, 64, 24, base, None) == E["shape"]     # the rank in steps of 16
    assert down(base, base, _lib.BF16, 0, 64, 16, base, None) == E["shape"]
    assert down(base, None, _lib.BF16, 4, 64, 16, base, None) == E["null"]
    assert down(base, base + 8, _lib.BF16, 4, 64, 16, base, None) == E["align"]
    # the two halves of the large-M call apart: which shapes have a prepared copy, and the checks of both calls
    nbytes = lib.mfq_qmm_t_prepared_bytes
    assert nbytes(3072, 3072, 4) == 3072 * 3072 * 2 and nbytes(3208, 512, 8) == 3216 * 512 * 2
    assert nbytes(3072, 3072, 5) == 3072 * 3072 * 2     # 3, 5 and 6 bits have the same copy
    assert nbytes(3072, 3072, 7) == 0 and nbytes(3072, 192, 4) == 0 and nbytes(3076, 512, 4) == 0 and nbytes(0, 512, 4) == 0
    prep = lib.mfq_qmm_t_prepare
    assert prep(base, base, base, _lib.F32, 64, 256, 64, 4, base, None) == E["dtype"]
    assert prep(base, base, base, _lib.BF16, 64, 256, 48, 4, base, None) == E["group"]
    assert prep(base, base, base, _lib.BF16, 64, 250, 64, 4, base, None) == E["shape"]
    assert prep(base, base, None, _lib.BF16, 64, 256, 64, 4, base, None) == E["null"]
    assert prep(base, base, base, _lib.BF16, 64, 256, 64, 4, base + 8, None) == E["align"]
    assert prep(base, base, base, _lib.BF16, 64, 192, 64, 4, base, None) == E["unsupported"]   # K not whole pairs of steps
    prepared = lib.mfq_qmm_t_prepared
    assert prepared(base, _lib.F32, 4, 256, base, None, 64, base, None, 0, None) == E["dtype"]
    assert prepared(base, _lib.BF16, 0, 256, base, None, 64, base, None, 0, None) == E["shape"]
    assert prepared(base, _lib.BF16, 4, 256, None, None, 64, base, None, 0, None) == E["null"]
    assert prepared(base, _lib.BF16, 4, 256, base, None, 64, base + 4, None, 0, None) == E["align"]
    assert prepared(base, _lib.BF16, 4, 192, base, None, 64, base, None, 0, None) == E["unsupported"]
    assert lib.mfq_qmm_t_prepared_workspace_bytes(4, 192, 64) == 0
    # the matvec with the activation inside: one row of 16-bit x, 4 or 8 bits, rows the one-row kernel takes
    silu = lib.mfq_qmv_silu

    def call_silu(x=base, xd=_lib.BF16, M=1, K=3072, wq=base, s=base, b=base, sd=_lib.BF16, N=64, gs=64, bits=8,
                  y=base, yd=_lib.BF16):
        return silu(x, xd, M, K, wq, s, b, sd, None, N, gs, bits, y, yd, None)

    assert call_silu(xd=_lib.F32, sd=_lib.F32) == E["dtype"]
    assert call_silu(xd=_lib.F16) == E["dtype"]
    assert call_silu(yd=_lib.F16) == E["dtype"]
    assert call_silu(K=3000) == E["shape"]
    assert call_silu(N=0) == E["shape"]
    assert call_silu(gs=48) == E["group"]
    assert call_silu(bits=7) == E["bits"]
    assert call_silu(x=None) == E["null"]
    assert call_silu(wq=base + 4) == E["align"]
    assert call_silu(bits=5) == E["unsupported"]
    assert call_silu(K=8192) == E["unsupported"]            # 8 KiB of 8-bit codes per row
    assert call_silu(K=8192, bits=4) == E["unsupported"]    # 4 KiB of 4-bit codes per row
    assert call_silu(M=0) == E["shape"]
    assert call_silu(M=5) == E["unsupported"]               # more rows than the fused kernels take
    assert call_silu(M=3, N=66) == E["unsupported"]         # the four-rows kernel wants whole quads of weight rows
    assert call_silu(M=2, K=8192, bits=4) == E["unsupported"]


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from mflux_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libmfq.so"))
    with pytest.raises(ImportError, match="no CPU or PyTorch fallback"):
        _lib.load()


def test_torch_ops_are_registered_and_refuse_cpu_tensors():
    """csrc/torch_ops.cpp: every op mflux_amd.core calls exists under
    torch.ops.mfq, only for the HIP backend (a CPU tensor is refused by the
    dispatcher: there is nothing to fall back to)."""
    import torch

    from mflux_amd import _lib

    ops = _lib.ops()
    for name in ("quantize_affine", "dequantize_affine", "dequantize_rows", "qmm_t", "qmv_silu", "low_rank_add_", "low_rank_down"):
        assert hasattr(ops, name), name
    with pytest.raises(NotImplementedError, match="CPU"):
        ops.quantize_affine(torch.zeros(2, 64, dtype=torch.bfloat16), 64, 4)
    with pytest.raises(NotImplementedError, match="CPU"):
        ops.qmm_t(torch.zeros(2, 64, dtype=torch.bfloat16), torch.zeros(4, 8, dtype=torch.int32).view(torch.uint32),
                  torch.zeros(4, 1, dtype=torch.bfloat16), torch.zeros(4, 1, dtype=torch.bfloat16), None, 64, 4,
                  torch.bfloat16, None, None)


def test_abi_validation_clean_under_host_sanitizers():
    """The C ABI's argument validation (csrc/abi.hip, host side) under
    AddressSanitizer and UndefinedBehaviorSanitizer: every refusal of
    tests/abi_sanitize_check.cpp comes back with its status and no finding."""
    from mflux_amd import _build

    assert "every refusal clean" in _build.sanitize_abi()


def test_generated_code_of_the_assembly_matrix_kernels():
    """The two-kernel GEMM states its matrix instruction as assembly (result tied
    to the addend), which hides it from the compiler's hazard recognizer; the
    build therefore refuses generated code that touches an accumulation register
    too soon after a matrix instruction wrote it, adds to one too soon after a
    write, waits for its newest loads inside the k loop, or spills more than a
    few dozen registers.  The check runs here on a fresh compile: eighteen kernels
    (two types x plain / with epilogue / with low-rank update x with / without
    the K cut, plain / with update on 192-column tiles, and the one whose
    deferred stores add a bias), all clean."""
    from mflux_amd import _build

    assert _build.check_generated_code("qmm_frag.hip") == 18


def _listing(blocks, spills=0):
    """A synthetic assembly listing of one kernel, `demo_gemm_kernel`, in the
    form the compiler prints: label lines, one instruction per line, the
    .Lfunc_end marker and the metadata entry with the spill count."""
    name = "_Z16demo_gemm_kernelv"
    lines = [f"{name}:"]
    for label, ins in blocks:
        if label:
            lines.append(f"{label}:")
        lines += [f"\t{i}" for i in ins]
    lines += [".Lfunc_end0:", "  - .name:           " + name, f"    .vgpr_spill_count: {spills}", ""]
    return "\n".join(lines)


def test_listing_check_follows_branches():
    """The distance between a matrix instruction and a read of its accumulator is
    measured along the control flow, back edges included, with an s_nop counted
    by its wait states: a loop whose head reads a register that the loop's last
    matrix instruction wrote is refused although the two lie hundreds of lines
    apart in the listing, and accepted once the wait states are stated."""
    from mflux_amd import _build

    mfma = "v_mfma_f32_16x16x32_bf16 a[0:3], v[0:3], v[4:7], a[0:3]"
    other = "v_mfma_f32_16x16x32_bf16 a[4:7], v[0:3], v[4:7], a[4:7]"
    filler = ["v_add_u32_e32 v9, v9, v9"] * 40
    head_bad = ["v_accvgpr_read_b32 v8, a1"] + filler
    tail = [other] * 3 + [mfma, "s_cmp_lg_u32 s0, 0", "s_cbranch_scc1 .LBB0_1"]
    end = [".LBB0_3", ["s_endpgm"]]
    # straight down the listing the read is 40-odd instructions behind every matrix instruction; over the
    # back edge it is 3 behind the one that writes a[0:3]
    bad = _listing([("", filler), (".LBB0_1", head_bad), (".LBB0_2", filler + tail), end])
    with pytest.raises(RuntimeError, match="touches a1 within 24 wait states"):
        _build.check_listing(bad, "demo_gemm_kernel")
    good = _listing([("", filler), (".LBB0_1", ["s_nop 15", "s_nop 15"] + head_bad), (".LBB0_2", filler + tail), end])
    assert _build.check_listing(good, "demo_gemm_kernel") == 1
    # a short block between the two does not hide the hazard either
    hop = _listing([("", filler), (".LBB0_1", head_bad), (".LBB0_2", filler + tail[:-1] + ["s_cbranch_scc1 .LBB0_4"]),
                    end, (".LBB0_4", ["s_mov_b32 s1, 0", "s_branch .LBB0_1"])])
    with pytest.raises(RuntimeError, match="touches a1"):
        _build.check_listing(hop, "demo_gemm_kernel")


def test_listing_check_refusals():
    """The other refusals on synthetic listings: an addend written from outside
    the matrix pipeline right in front of the instruction, a k loop that waits
    for its newest loads, too many spills, a listing without the kernel."""
    from mflux_amd import _build

    mfma = "v_mfma_f32_16x16x32_bf16 a[0:3], v[0:3], v[4:7], a[0:3]"
    end = (".LBB0_9", ["s_endpgm"])
    with pytest.raises(RuntimeError, match="adds to a\\[0:3\\] within 4"):
        _build.check_listing(_listing([("", ["v_accvgpr_write_b32 a2, v1", "s_nop 1", mfma]), end]), "demo_gemm_kernel")
    assert _build.check_listing(_listing([("", ["v_accvgpr_write_b32 a2, v1", "s_nop 3", mfma]), end]),
                                "demo_gemm_kernel") == 1
    loop = [mfma] * 64 + ["s_waitcnt vmcnt(2)"] + [mfma] * 64
    with pytest.raises(RuntimeError, match="vmcnt\\(2\\) inside its k loop"):
        _build.check_listing(_listing([("", loop), end]), "demo_gemm_kernel")
    with pytest.raises(RuntimeError, match="spills 49"):
        _build.check_listing(_listing([("", [mfma]), end], spills=49), "demo_gemm_kernel")
    with pytest.raises(RuntimeError, match="no kernel named"):
        _build.check_listing(_listing([("", [mfma]), end]), "other_kernel")
