"""TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.

numpy restatement of MLX's group-wise affine quantization, written
independently of ``mlx_affine.c`` (vectorised over groups instead of the
scalar loops of MLX's CPU kernel) so that the two can be checked against each
other, plus the float64 matmul oracle.

Reference call sites this stands in for: ``nn.quantize`` at
src/mflux/models/common/weights/loading/weight_applier.py:43,46,103 (which
reaches ``mx.quantize`` through ``Linear.to_quantized``) and every
``QuantizedLinear.__call__`` such as
src/mflux/models/flux/model/flux_transformer/single_transformer_block.py:53,57
(which reaches ``mx.quantized_matmul(..., transpose=True)``).  The arithmetic
is MLX's (third-party, pinned 0.30.3 / 0.31.0 by pyproject.toml:69-70, sources
not in the reference tree): mlx/backend/cpu/quantized.cpp ``quantize`` and
mlx/ops.cpp ``dequantize`` / ``quantized_matmul``.

Parity status: ``quantize`` is "parity unpinned" against MLX itself (no golden
vector exists in the reference and MLX cannot run here); it is pinned by
hand-computed known answers, algebraic invariants and the C restatement.
``dequantize_exact`` and ``quantized_matmul_f64`` are pinned by definition
(``q*s+b`` and a textbook matrix product).

Only tests/, ``__graft_entry__.smoke()`` and bench.py's ``cpu_baseline`` leg
may import this module.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

EPS = np.float32(1e-7)

F32, F16, BF16 = 0, 1, 2


# --------------------------------------------------------------------------
# bfloat16 <-> float32 on raw uint16 bit patterns (numpy has no bfloat16)
# --------------------------------------------------------------------------
def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round to nearest even, as MLX's bfloat16 conversion does."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    rounded = u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))
    out = (rounded >> np.uint32(16)).astype(np.uint16)
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    if nan.any():
        out = np.where(nan, ((u >> np.uint32(16)) | np.uint32(0x40)).astype(np.uint16), out)
    return out


def _to_f32(w: np.ndarray, dtype: int) -> np.ndarray:
    if dtype == BF16:
        return bf16_bits_to_f32(w)
    if dtype == F16:
        return np.ascontiguousarray(w).view(np.float16).astype(np.float32)
    return np.ascontiguousarray(w, dtype=np.float32)


def _from_f32(x: np.ndarray, dtype: int) -> np.ndarray:
    if dtype == BF16:
        return f32_to_bf16_bits(x)
    if dtype == F16:
        return x.astype(np.float16).view(np.uint16)
    return x.astype(np.float32)


def silu_bits(x: np.ndarray, dtype: int = BF16) -> np.ndarray:
    """MLX's ``nn.silu`` on raw 16-bit storage: ``x * sigmoid(x)`` as two array
    operations, each rounded to ``dtype`` (python/mlx/nn/layers/activations.py,
    ``silu``; reached from src/mflux/models/flux/model/flux_transformer/
    ada_layer_norm_zero.py:12).  The sigmoid is evaluated in float64, with the
    float32 range of the exponential.

    Parity unpinned against MLX itself (its sigmoid kernel's own rounding is not
    available here); pinned by tests/test_oracle.py against PyTorch's CPU
    evaluation of the same two operations, closed-form values and limits."""
    xf = _to_f32(x, dtype).astype(np.float64)
    with np.errstate(over="ignore"):
        e = np.exp(-xf)
    e = np.where(e > float(np.finfo(np.float32).max), np.inf, e)  # the exponential is a float32 one: x < -88.7 overflows
    sg = 1.0 / (1.0 + e)
    sg16 = _to_f32(_from_f32(sg.astype(np.float32), dtype), dtype).astype(np.float64)
    with np.errstate(invalid="ignore"):
        prod = (xf * sg16).astype(np.float32)  # exact: two 8- or 11-bit significands
    return _from_f32(prod, dtype)


def _check(group_size: int, bits: int) -> None:
    if group_size not in (32, 64, 128):
        raise ValueError(f"group_size {group_size} not supported")
    if bits not in (2, 3, 4, 5, 6, 8):
        raise ValueError(f"bits {bits} not supported")


# --------------------------------------------------------------------------
# quantize / dequantize
# --------------------------------------------------------------------------
def quantize(w: np.ndarray, dtype: int = BF16, group_size: int = 64, bits: int = 4):
    """w: [..., K] raw storage (uint16 bit patterns for bf16/f16, float32 for
    f32).  Returns (wq uint32 [..., K*bits/32], scales, biases [..., K/gs]) with
    scales/biases in the same raw storage as w."""
    _check(group_size, bits)
    if w.ndim < 2:
        raise ValueError("quantize needs a matrix (ndim >= 2)")
    K = w.shape[-1]
    if K % group_size:
        raise ValueError(f"last dimension {K} is not divisible by group_size {group_size}")
    lead = w.shape[:-1]
    f = _to_f32(w, dtype).reshape(-1, group_size)
    n_bins = np.float32((1 << bits) - 1)
    with np.errstate(all="ignore"):
        w_min = f.min(axis=1)
        w_max = f.max(axis=1)
        mask = np.abs(w_min) > np.abs(w_max)
        scale = np.maximum((w_max - w_min) / n_bins, EPS)
        scale = np.where(mask, scale, -scale).astype(np.float32)
        edge = np.where(mask, w_min, w_max).astype(np.float32)
        q0 = np.rint(edge / scale)
        nz = q0 != 0
        scale = np.where(nz, edge / np.where(nz, q0, np.float32(1)), scale).astype(np.float32)
        bias = np.where(nz, edge, np.float32(0)).astype(np.float32)
        codes = np.rint((f - bias[:, None]) / scale[:, None])
        codes = np.minimum(np.maximum(codes, np.float32(0)), n_bins).astype(np.uint32)
    words = pack_bitstream(codes.reshape(-1, K), bits)
    wq = words.reshape(*lead, K * bits // 32)
    scales = _from_f32(scale, dtype).reshape(*lead, K // group_size)
    biases = _from_f32(bias, dtype).reshape(*lead, K // group_size)
    return wq, scales, biases


def pack_bitstream(codes: np.ndarray, bits: int) -> np.ndarray:
    """codes [R, K] -> uint32 [R, K*bits/32]: every row is one little-endian bit
    stream in which code i occupies bits [i*bits, (i+1)*bits).  For 2, 4 and 8
    bits that is MLX's "element i of a word at bit offset i*bits"; for 3, 5 and
    6 bits it is MLX's byte packs (8 codes in 3 bytes, 8 in 5, 4 in 3), whose
    boundaries fall on whole bytes of the same stream."""
    codes = np.ascontiguousarray(codes, dtype=np.uint32)
    rows, K = codes.shape
    bit = ((codes[:, :, None] >> np.arange(bits, dtype=np.uint32)) & np.uint32(1)).astype(np.uint8)
    stream = np.packbits(bit.reshape(rows, K * bits), axis=1, bitorder="little")
    return np.ascontiguousarray(stream).view(np.uint32).reshape(rows, K * bits // 32)


def unpack_codes(wq: np.ndarray, bits: int) -> np.ndarray:
    """uint32 [..., W] -> uint32 codes [..., W*32/bits], code i of a row at bit
    offset i*bits of the row's little-endian bit stream."""
    wq = np.ascontiguousarray(wq, dtype=np.uint32)
    lead, W = wq.shape[:-1], wq.shape[-1]
    stream = np.unpackbits(wq.reshape(-1, W).view(np.uint8), axis=1, bitorder="little")
    n = W * 32 // bits
    bit = stream[:, :n * bits].reshape(-1, n, bits).astype(np.uint32)
    codes = (bit << np.arange(bits, dtype=np.uint32)).sum(axis=2, dtype=np.uint32)
    return codes.reshape(*lead, n)


def dequantize_exact(wq, scales, biases, dtype: int = BF16, group_size: int = 64, bits: int = 4) -> np.ndarray:
    """float64 code*scale+bias; exact (no rounding) for bf16/f16 scales."""
    _check(group_size, bits)
    codes = unpack_codes(wq, bits).astype(np.float64)
    s = np.repeat(_to_f32(scales, dtype).astype(np.float64), group_size, axis=-1)
    b = np.repeat(_to_f32(biases, dtype).astype(np.float64), group_size, axis=-1)
    return codes * s + b


def dequantize(wq, scales, biases, dtype: int = BF16, group_size: int = 64, bits: int = 4) -> np.ndarray:
    """MLX-style dequantize in the storage type: product rounded to the
    storage type, then the sum rounded again.  Returns raw storage."""
    _check(group_size, bits)
    codes = unpack_codes(wq, bits).astype(np.float32)
    s = np.repeat(_to_f32(scales, dtype), group_size, axis=-1)
    b = np.repeat(_to_f32(biases, dtype), group_size, axis=-1)
    prod = _to_f32(_from_f32(codes * s, dtype), dtype)
    return _from_f32(prod + b, dtype)


def quantized_matmul_f64(x_f64: np.ndarray, wq, scales, biases, dtype: int = BF16,
                         group_size: int = 64, bits: int = 4, bias_f64=None) -> np.ndarray:
    """y = x @ dequantize_exact(w).T (+ bias) in float64: the matmul oracle."""
    w = dequantize_exact(wq, scales, biases, dtype, group_size, bits)
    y = np.asarray(x_f64, dtype=np.float64) @ w.T
    if bias_f64 is not None:
        y = y + np.asarray(bias_f64, dtype=np.float64)
    return y


# --------------------------------------------------------------------------
# ctypes binding of the C restatement
# --------------------------------------------------------------------------
_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmlx_affine_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s", "all"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


def clib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        lib = ctypes.CDLL(_LIB_PATH)
        sz, vp, i32 = ctypes.c_size_t, ctypes.c_void_p, ctypes.c_int
        lib.mlxo_quantize.argtypes = [vp, i32, sz, i32, i32, vp, vp, vp]
        lib.mlxo_dequantize.argtypes = [vp, vp, vp, i32, sz, i32, i32, vp, i32]
        lib.mlxo_dequantize_f64.argtypes = [vp, vp, vp, i32, sz, i32, i32, vp]
        lib.mlxo_qmm_t_f32acc.argtypes = [vp, i32, sz, sz, vp, vp, vp, i32, vp, sz, i32, i32, vp, i32, i32]
        lib.mlxo_qmm_t_tacc.argtypes = [vp, sz, sz, vp, vp, vp, i32, sz, i32, i32, vp]
        for f in (lib.mlxo_quantize, lib.mlxo_dequantize, lib.mlxo_dequantize_f64,
                  lib.mlxo_qmm_t_f32acc, lib.mlxo_qmm_t_tacc, lib.mlxo_num_threads):
            f.restype = i32
        _lib = lib
    return _lib


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def _storage(dtype: int):
    return np.float32 if dtype == F32 else np.uint16


def c_quantize(w: np.ndarray, dtype: int = BF16, group_size: int = 64, bits: int = 4):
    w = np.ascontiguousarray(w, dtype=_storage(dtype))
    K = w.shape[-1]
    if w.ndim < 2 or K % group_size:
        raise ValueError(f"quantize needs ndim >= 2 and a last dimension divisible by {group_size}, got {w.shape}")
    lead = w.shape[:-1]
    wq = np.empty((*lead, K * bits // 32), dtype=np.uint32)
    scales = np.empty((*lead, K // group_size), dtype=_storage(dtype))
    biases = np.empty_like(scales)
    rc = clib().mlxo_quantize(_ptr(w), dtype, w.size, group_size, bits, _ptr(wq), _ptr(scales), _ptr(biases))
    if rc:
        raise ValueError(f"mlxo_quantize failed with {rc}")
    return wq, scales, biases


def c_dequantize(wq, scales, biases, dtype: int = BF16, group_size: int = 64, bits: int = 4, out_dtype=None):
    out_dtype = dtype if out_dtype is None else out_dtype
    wq = np.ascontiguousarray(wq, dtype=np.uint32)
    scales = np.ascontiguousarray(scales)
    biases = np.ascontiguousarray(biases)
    n = wq.size * 32 // bits
    out = np.empty((*wq.shape[:-1], wq.shape[-1] * 32 // bits), dtype=_storage(out_dtype))
    rc = clib().mlxo_dequantize(_ptr(wq), _ptr(scales), _ptr(biases), dtype, n, group_size, bits, _ptr(out), out_dtype)
    if rc:
        raise ValueError(f"mlxo_dequantize failed with {rc}")
    return out


def c_dequantize_f64(wq, scales, biases, dtype: int = BF16, group_size: int = 64, bits: int = 4):
    wq = np.ascontiguousarray(wq, dtype=np.uint32)
    scales = np.ascontiguousarray(scales)
    biases = np.ascontiguousarray(biases)
    n = wq.size * 32 // bits
    out = np.empty((*wq.shape[:-1], wq.shape[-1] * 32 // bits), dtype=np.float64)
    rc = clib().mlxo_dequantize_f64(_ptr(wq), _ptr(scales), _ptr(biases), dtype, n, group_size, bits, _ptr(out))
    if rc:
        raise ValueError(f"mlxo_dequantize_f64 failed with {rc}")
    return out


def c_qmm_t(x, x_dtype, wq, scales, biases, sb_dtype=BF16, bias=None, group_size=64, bits=4,
            y_dtype=None, threads=0, accumulate="f32"):
    """x: [M, K] raw storage.  Returns y [M, N] raw storage of y_dtype."""
    x = np.ascontiguousarray(x, dtype=_storage(x_dtype))
    wq = np.ascontiguousarray(wq, dtype=np.uint32)
    scales = np.ascontiguousarray(scales)
    biases = np.ascontiguousarray(biases)
    M, K = x.shape
    N = wq.shape[0]
    y_dtype = sb_dtype if y_dtype is None else y_dtype
    y = np.empty((M, N), dtype=_storage(y_dtype))
    if accumulate == "f32":
        bias_arr = np.ascontiguousarray(bias) if bias is not None else None
        bp = _ptr(bias_arr) if bias_arr is not None else None
        rc = clib().mlxo_qmm_t_f32acc(_ptr(x), x_dtype, M, K, _ptr(wq), _ptr(scales), _ptr(biases), sb_dtype,
                                      bp, N, group_size, bits, _ptr(y), y_dtype, threads)
    else:
        assert x_dtype == sb_dtype == y_dtype and bias is None
        rc = clib().mlxo_qmm_t_tacc(_ptr(x), M, K, _ptr(wq), _ptr(scales), _ptr(biases), sb_dtype,
                                    N, group_size, bits, _ptr(y))
    if rc:
        raise ValueError(f"mlxo_qmm_t failed with {rc}")
    return y


def num_threads() -> int:
    return int(clib().mlxo_num_threads())
