"""ctypes binding of libmfq.so (the C ABI declared in include/mfq.h).

There is no fallback: if the library has not been built, or a call returns an
error code, an exception is raised.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libmfq.so")

F32, F16, BF16 = 0, 1, 2
MFQ_EUNSUPPORTED = -8  # no kernel for this combination of arguments
EPILOGUE_GELU, EPILOGUE_GATE_RESIDUAL, EPILOGUE_SWIGLU = 1, 2, 3
MFQ_ESCRATCH = -9  # mfq_qmm_t_static: the K split needs more than the built-in buffer

# every symbol include/mfq.h declares, with its ctypes signature
_I64, _INT, _PTR = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p
SIGNATURES = {
    "mfq_version": (_INT, []),
    "mfq_strerror": (ctypes.c_char_p, [_INT]),
    "mfq_quantize_affine": (_INT, [_PTR, _INT, _I64, _I64, _INT, _INT, _PTR, _PTR, _PTR, _PTR]),
    "mfq_dequantize_affine": (_INT, [_PTR, _PTR, _PTR, _INT, _I64, _I64, _INT, _INT, _PTR, _INT, _PTR]),
    "mfq_dequantize_rows": (_INT, [_PTR, _PTR, _PTR, _INT, _PTR, _I64, _I64, _I64, _INT, _INT, _PTR, _INT, _PTR]),
    "mfq_qmm_t": (_INT, [_PTR, _INT, _I64, _I64, _PTR, _PTR, _PTR, _INT, _PTR, _I64, _INT, _INT, _PTR, _INT, _PTR]),
    "mfq_qmm_t_epilogue": (_INT, [_PTR, _INT, _I64, _I64, _PTR, _PTR, _PTR, _INT, _PTR, _I64, _INT, _INT, _INT, _PTR, _PTR,
                                  _I64, _PTR, _INT, _PTR, ctypes.c_size_t, _PTR]),
    "mfq_qmm_n": (_INT, [_PTR, _INT, _I64, _I64, _PTR, _PTR, _PTR, _INT, _I64, _INT, _INT, _PTR, _INT, _PTR]),
    "mfq_qmm_n_workspace_bytes": (ctypes.c_size_t, [_I64, _I64, _I64, _INT, _INT]),
    "mfq_qmm_n_ws": (_INT, [_PTR, _INT, _I64, _I64, _PTR, _PTR, _PTR, _INT, _I64, _INT, _INT, _PTR, _INT, _PTR,
                            ctypes.c_size_t, _PTR]),
    "mfq_qmm_t_workspace_bytes": (ctypes.c_size_t, [_I64, _I64, _I64, _INT, _INT]),
    "mfq_qmm_t_ws": (_INT, [_PTR, _INT, _I64, _I64, _PTR, _PTR, _PTR, _INT, _PTR, _I64, _INT, _INT, _PTR, _INT, _PTR,
                            ctypes.c_size_t, _PTR]),
    "mfq_qmm_t_prepared_bytes": (ctypes.c_size_t, [_I64, _I64, _INT]),
    "mfq_qmm_t_prepare": (_INT, [_PTR, _PTR, _PTR, _INT, _I64, _I64, _INT, _INT, _PTR, _PTR]),
    "mfq_qmm_t_prepared_workspace_bytes": (ctypes.c_size_t, [_I64, _I64, _I64]),
    "mfq_qmm_t_prepared": (_INT, [_PTR, _INT, _I64, _I64, _PTR, _PTR, _I64, _PTR, _PTR, ctypes.c_size_t, _PTR]),
    "mfq_qmm_t_static": (_INT, [_PTR, _INT, _I64, _I64, _PTR, _PTR, _PTR, _INT, _PTR, _I64, _INT, _INT, _PTR, _INT, _PTR]),
    "mfq_qmm_t_low_rank": (_INT, [_PTR, _INT, _I64, _I64, _PTR, _PTR, _PTR, _INT, _PTR, _I64, _INT, _INT, _PTR, _PTR,
                                  _I64, _PTR, _INT, _PTR, ctypes.c_size_t, _PTR]),
    "mfq_qmv_silu": (_INT, [_PTR, _INT, _I64, _I64, _PTR, _PTR, _PTR, _INT, _PTR, _I64, _INT, _INT, _PTR, _INT, _PTR]),
    "mfq_layer_norm_modulate": (_INT, [_PTR, _INT, _I64, _I64, _PTR, _PTR, _I64, ctypes.c_float, _PTR, _PTR]),
    "mfq_low_rank_down": (_INT, [_PTR, _PTR, _INT, _I64, _I64, _I64, _PTR, _PTR]),
    "mfq_low_rank_add": (_INT, [_PTR, _PTR, _INT, _I64, _I64, _I64, _PTR, _INT, _PTR]),
}

_lib = None


class MfqError(RuntimeError):
    """A libmfq entry point returned a negative status."""

    def __init__(self, fn: str, status: int, message: str):
        super().__init__(f"{fn} failed: {message} (status {status})")
        self.status = status


def load() -> ctypes.CDLL:
    """Loads libmfq.so from the source tree; raises if it is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m mflux_amd._build` "
                "(there is no CPU or PyTorch fallback for the quantized kernels)"
            )
        lib = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    return _lib


OPS_PATH = os.path.join(_HERE, "csrc", "libmfq_torch.so")
_ops = None


def ops():
    """``torch.ops.mfq``: the ops of csrc/torch_ops.cpp over the same libmfq.so
    (its RUNPATH is its own directory).  Raises if either library is not built."""
    global _ops
    if _ops is None:
        import torch

        load()
        if not os.path.exists(OPS_PATH):
            raise ImportError(f"{OPS_PATH} is missing: build it with `python -m mflux_amd._build`")
        torch.ops.load_library(OPS_PATH)
        _ops = torch.ops.mfq
    return _ops


def check(fn: str, status: int) -> None:
    if status != 0:
        raise MfqError(fn, status, load().mfq_strerror(status).decode())
