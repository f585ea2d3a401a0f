"""Functional API: ``quantize``, ``dequantize``, ``quantized_matmul``.

Same names, argument meaning and error behaviour as ``mx.quantize``,
``mx.dequantize`` and ``mx.quantized_matmul`` (mode ``"affine"``), which is
where mflux's quantized linears land: ``nn.quantize`` at
src/mflux/models/common/weights/loading/weight_applier.py:43,46,103 and every
quantized ``nn.Linear`` call such as
src/mflux/models/flux/model/flux_transformer/single_transformer_block.py:53,57.

Tensors are torch tensors on a HIP device; torch only provides the device
memory and the stream, the arithmetic is libmfq's hand-written kernels, reached
through the ``torch.ops.mfq`` ops of csrc/torch_ops.cpp (a thin C++ layer over
the C ABI of include/mfq.h).
"""
from __future__ import annotations

import torch

from . import _lib

_DTYPE_CODE = {torch.float32: _lib.F32, torch.float16: _lib.F16, torch.bfloat16: _lib.BF16}
SUPPORTED_GROUP_SIZES = (32, 64, 128)
MLX_BITS = (2, 3, 4, 5, 6, 8)  # what mx.quantize accepts
SUPPORTED_BITS = (3, 4, 5, 6, 8)  # what quantize / dequantize have kernels for
MATMUL_KERNEL_BITS = (4, 8)  # what the SiLU-fused matvec kernels take


def _check_mode(fn: str, mode: str) -> None:
    if mode != "affine":
        raise ValueError(f"[{fn}] Invalid quantization mode '{mode}': this build implements 'affine' only.")


def _check_group_bits(fn: str, group_size: int, bits: int) -> None:
    if group_size not in SUPPORTED_GROUP_SIZES:
        raise ValueError(
            f"[{fn}] The requested group size {group_size} is not supported. "
            "The supported group sizes are 32, 64, and 128."
        )
    if bits not in MLX_BITS:
        raise ValueError(
            f"[{fn}] The requested number of bits {bits} is not supported. "
            "The supported bits are 2, 3, 4, 5, 6 and 8."
        )
    if bits not in SUPPORTED_BITS:
        raise ValueError(f"[{fn}] {bits}-bit packing is not implemented in this build (3, 4, 5, 6 and 8 are).")


def _require_hip(fn: str, t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(
            f"[{fn}] `{name}` lives on {t.device}; the mfq kernels run on a HIP device only "
            "and there is no CPU fallback."
        )


def quantize(w: torch.Tensor, group_size: int = 64, bits: int = 4, mode: str = "affine"):
    """Group-wise affine quantization of the last axis of ``w``.

    Returns ``(w_q, scales, biases)``: ``w_q`` uint32 ``[..., K*bits/32]`` with
    element ``i`` of each word at bit offset ``i*bits``; ``scales``/``biases`` of
    ``w``'s dtype, ``[..., K/group_size]``.  Bit-identical to the restatement of
    MLX's CPU algorithm in oracle/mlx_affine.c (parity with MLX itself is
    unpinned: it cannot be run here).
    """
    _check_mode("quantize", mode)
    _check_group_bits("quantize", group_size, bits)
    if w.dtype not in _DTYPE_CODE:
        raise ValueError(f"[quantize] Only floating point inputs are supported but got {w.dtype}.")
    if w.ndim < 2:
        raise ValueError(
            f"[quantize] The matrix to be quantized must have at least 2 dimension but it has only {w.ndim}."
        )
    K = w.shape[-1]
    if K % group_size != 0:
        raise ValueError(
            "[quantize] The last dimension of the matrix needs to be divisible by the quantization "
            f"group size {group_size}. However the provided matrix has shape {tuple(w.shape)}"
        )
    _require_hip("quantize", w, "w")
    lead = tuple(w.shape[:-1])
    wq, scales, biases = _lib.ops().quantize_affine(w.reshape(-1, K).contiguous(), group_size, bits)
    return wq.reshape(*lead, -1), scales.reshape(*lead, -1), biases.reshape(*lead, -1)


def _check_packed(fn: str, w: torch.Tensor, scales: torch.Tensor, biases: torch.Tensor, group_size: int, bits: int):
    if w.dtype != torch.uint32:
        raise ValueError(f"[{fn}] The weight matrix should be uint32 but received {w.dtype}")
    if scales.shape != biases.shape:
        raise ValueError(f"[{fn}] Scales and biases should have the same shape. Received scales with shape "
                         f"{tuple(scales.shape)} and biases with {tuple(biases.shape)}")
    if scales.dtype != biases.dtype or scales.dtype not in _DTYPE_CODE:
        raise ValueError(f"[{fn}] Scales and biases must share a floating point dtype, got {scales.dtype} "
                         f"and {biases.dtype}")
    if w.ndim < 2 or w.shape[:-1] != scales.shape[:-1]:
        raise ValueError(f"[{fn}] Weight, scales and biases should have the same batch shape. Received weight "
                         f"with shape {tuple(w.shape)}, scales with {tuple(scales.shape)}")
    if w.shape[-1] * 32 // bits != scales.shape[-1] * group_size:
        raise ValueError(
            f"[{fn}] The shapes of the weight and scales are incompatible based on bits and group_size. "
            f"w.shape() == {tuple(w.shape)} and scales.shape() == {tuple(scales.shape)} "
            f"with group_size={group_size} and bits={bits}"
        )


def _rows2d(t: torch.Tensor) -> torch.Tensor:
    return t.reshape(-1, t.shape[-1]).contiguous()


def dequantize(w: torch.Tensor, scales: torch.Tensor, biases: torch.Tensor, group_size: int = 64, bits: int = 4,
               mode: str = "affine", dtype: torch.dtype | None = None) -> torch.Tensor:
    """``code * scale + bias`` in ``dtype`` (default: the dtype of ``scales``),
    evaluated as ``mx.dequantize`` does: the product is rounded to ``dtype``, then
    the sum is."""
    _check_mode("dequantize", mode)
    _check_group_bits("dequantize", group_size, bits)
    _check_packed("dequantize", w, scales, biases, group_size, bits)
    _require_hip("dequantize", w, "w")
    out_dtype = scales.dtype if dtype is None else dtype
    if out_dtype not in (scales.dtype, torch.float32):
        raise ValueError(f"[dequantize] Output dtype must be {scales.dtype} or float32, got {out_dtype}")
    K = w.shape[-1] * 32 // bits
    out = _lib.ops().dequantize_affine(_rows2d(w), _rows2d(scales), _rows2d(biases), group_size, bits, out_dtype)
    return out.reshape(*w.shape[:-1], K)


def dequantize_rows(w: torch.Tensor, scales: torch.Tensor, biases: torch.Tensor, indices: torch.Tensor,
                    group_size: int = 64, bits: int = 4, mode: str = "affine",
                    dtype: torch.dtype | None = None) -> torch.Tensor:
    """``dequantize(w[indices], scales[indices], biases[indices])`` in one pass:
    the lookup of a quantized embedding table.  ``indices`` is an integer tensor
    of any shape; the result has shape ``indices.shape + (K,)``.  Negative
    indices count from the end; indices outside the table are clamped."""
    _check_mode("dequantize", mode)
    _check_group_bits("dequantize", group_size, bits)
    _check_packed("dequantize", w, scales, biases, group_size, bits)
    if w.ndim != 2:
        raise ValueError(f"[dequantize] a table to look rows up in must be 2-D, got shape {tuple(w.shape)}")
    if indices.dtype.is_floating_point or indices.dtype == torch.bool:
        raise ValueError(f"[dequantize] indices must be integers, got {indices.dtype}")
    _require_hip("dequantize", w, "w")
    out_dtype = scales.dtype if dtype is None else dtype
    if out_dtype not in (scales.dtype, torch.float32):
        raise ValueError(f"[dequantize] Output dtype must be {scales.dtype} or float32, got {out_dtype}")
    K = w.shape[1] * 32 // bits
    idx = indices.to(device=w.device, dtype=torch.int64).reshape(-1).contiguous()
    out = _lib.ops().dequantize_rows(w.contiguous(), scales.contiguous(), biases.contiguous(), idx, group_size, bits,
                                     out_dtype)
    return out.reshape(*indices.shape, K)


def _matmul_untransposed(x, w, scales, biases, group_size, bits):
    """``x @ dequantize(w)`` (``w`` packed ``[N, K*bits/32]``, ``x`` ``[..., N]``): the
    product MLX computes for ``transpose=False``, which is what the gradient of a
    quantized linear with respect to its input needs when a LoRA is trained on a
    quantized base (src/mflux/models/common/training/lora/target_injector.py:30-33
    wraps ``nn.QuantizedLinear`` in a trainable ``LoRALinear``).  One kernel
    (``mfq_qmm_n``): the weight tile is dequantised and transposed on its way
    into LDS; float32 ``x`` is rounded to the dtype of ``scales`` as for
    ``transpose=True``."""
    _check_packed("quantized_matmul", w, scales, biases, group_size, bits)
    if w.ndim != 2:
        raise NotImplementedError("[quantized_matmul] batched weights are not implemented in this build")
    if scales.dtype == torch.float32:
        raise NotImplementedError("[quantized_matmul] float32 scales are not implemented in this build")
    N = w.shape[0]
    K = w.shape[1] * 32 // bits
    if x.ndim < 1 or x.shape[-1] != N:
        raise ValueError(
            f"[quantized_matmul] Last dimension of first input with shape {tuple(x.shape)} does not match the "
            f"expanded quantized matrix ({N}, {K}) computed from shape {tuple(w.shape)} with "
            f"group_size={group_size}, bits={bits} and transpose=false"
        )
    _require_hip("quantized_matmul", x, "x")
    _require_hip("quantized_matmul", w, "w")
    out_dtype = torch.result_type(x, scales)
    lead = tuple(x.shape[:-1])
    x2 = x.reshape(-1, N).to(scales.dtype)
    w, scales, biases = w.contiguous(), scales.contiguous(), biases.contiguous()
    if N % 8:
        # the kernel reads x in 16-byte pieces: zero columns of x against zero rows of the weight add nothing
        pad = 8 - N % 8
        x2 = torch.nn.functional.pad(x2, (0, pad))
        w = torch.cat([w, w.new_zeros((pad, w.shape[1]))])
        scales = torch.cat([scales, scales.new_zeros((pad, scales.shape[1]))])
        biases = torch.cat([biases, biases.new_zeros((pad, biases.shape[1]))])
    if x2.shape[0] == 0:
        return torch.empty((*lead, K), dtype=out_dtype, device=x.device)
    y, ok = _lib.ops().qmm_n(x2.contiguous(), w, scales, biases, group_size, bits, out_dtype)
    if not ok:
        raise NotImplementedError(f"[quantized_matmul] no kernel for x {tuple(x.shape)} against a weight of "
                                  f"{N} x {K} with transpose=False (an operand exceeds 2 GiB)")
    return y.reshape(*lead, K)


class _QuantizedMatmulFunction(torch.autograd.Function):
    """Makes the fused forward differentiable with respect to ``x`` (and to a
    trainable ``bias``); the packed weight, scales and biases are constants."""

    @staticmethod
    def forward(ctx, x, w, scales, biases, bias, group_size, bits):
        ctx.save_for_backward(w, scales, biases)
        ctx.meta = (group_size, bits, x.dtype, bias is not None, bias.dtype if bias is not None else None)
        return _quantized_matmul_forward(x, w, scales, biases, group_size, bits, bias)

    @staticmethod
    def backward(ctx, grad_y):
        w, scales, biases = ctx.saved_tensors
        group_size, bits, x_dtype, has_bias, bias_dtype = ctx.meta
        grad_x = grad_bias = None
        if ctx.needs_input_grad[0]:
            grad_x = _matmul_untransposed(grad_y, w, scales, biases, group_size, bits).to(x_dtype)
        if has_bias and ctx.needs_input_grad[4]:
            grad_bias = grad_y.reshape(-1, grad_y.shape[-1]).sum(dim=0).to(bias_dtype)
        return grad_x, None, None, None, grad_bias, None, None


def quantized_matmul(x: torch.Tensor, w: torch.Tensor, scales: torch.Tensor, biases: torch.Tensor,
                     transpose: bool = True, group_size: int = 64, bits: int = 4, mode: str = "affine",
                     *, bias: torch.Tensor | None = None,
                     low_rank: tuple[torch.Tensor, torch.Tensor] | None = None) -> torch.Tensor:
    """``x @ dequantize(w).T`` (``transpose=True``) or ``x @ dequantize(w)``; see
    ``_quantized_matmul_forward``.  Differentiable with respect to ``x`` and
    ``bias``; ``low_rank`` (inference only) is described there."""
    _check_mode("quantized_matmul", mode)
    _check_group_bits("quantized_matmul", group_size, bits)
    if not transpose:
        if bias is not None or low_rank is not None:
            raise ValueError("[quantized_matmul] bias and low_rank are only fused for transpose=True")
        return _matmul_untransposed(x, w, scales, biases, group_size, bits)
    needs_grad = torch.is_grad_enabled() and (x.requires_grad or (bias is not None and bias.requires_grad))
    if needs_grad:
        if low_rank is not None:
            raise ValueError("[quantized_matmul] low_rank is not differentiable: add the LoRA branch as separate "
                             "matmuls when gradients are needed")
        return _QuantizedMatmulFunction.apply(x, w, scales, biases, bias, group_size, bits)
    return _quantized_matmul_forward(x, w, scales, biases, group_size, bits, bias, low_rank)



class PreparedWeights:
    """What :func:`prepare_weights` returns: the 16-bit copy (``data``, an opaque
    uint8 tensor) together with what it was made from -- the dtype of the values,
    the weight's ``output_dims`` x ``input_dims``, ``group_size`` and ``bits`` --
    so that :func:`quantized_matmul_prepared` can refuse an ``x`` of another dtype
    or width instead of multiplying it with bytes that mean something else (a
    bfloat16 and a float16 copy of one shape have the same size)."""

    __slots__ = ("data", "dtype", "output_dims", "input_dims", "group_size", "bits")

    def __init__(self, data, dtype, output_dims, input_dims, group_size, bits):
        self.data, self.dtype = data, dtype
        self.output_dims, self.input_dims = int(output_dims), int(input_dims)
        self.group_size, self.bits = int(group_size), int(bits)

    def numel(self) -> int:
        return self.data.numel()

    def __repr__(self) -> str:
        return (f"PreparedWeights({self.output_dims} x {self.input_dims}, {self.dtype}, group_size={self.group_size}, "
                f"bits={self.bits}, {self.data.numel()} bytes on {self.data.device})")


def prepare_weights(w: torch.Tensor, scales: torch.Tensor, biases: torch.Tensor, group_size: int = 64,
                    bits: int = 4) -> PreparedWeights | None:
    """The 16-bit copy of ``dequantize(w)`` that a large ``quantized_matmul``
    makes on every call, made once: for weights that do not change between calls
    and a caller with 2 bytes per weight of device memory to spare
    (``include/mfq.h``: ``mfq_qmm_t_prepare``).  Not part of MLX, which
    dequantises inside every ``mx.quantized_matmul``.  Returns a
    :class:`PreparedWeights` for ``quantized_matmul_prepared``, or ``None`` where
    the library has no such copy for the shape (``K`` not a multiple of 128,
    ``N`` not a multiple of 8).  The values are those every other kernel
    multiplies with: one rounding of ``fma(code, scale, bias)`` to the dtype of
    ``scales``."""
    _check_group_bits("prepare_weights", group_size, bits)
    _check_packed("prepare_weights", w, scales, biases, group_size, bits)
    if w.ndim != 2 or scales.dtype not in (torch.float16, torch.bfloat16):
        return None
    _require_hip("prepare_weights", w, "w")
    lib = _lib.load()
    N, K = w.shape[0], w.shape[1] * 32 // bits
    need = lib.mfq_qmm_t_prepared_bytes(N, K, bits)
    if need == 0:
        return None
    w, scales, biases = w.contiguous(), scales.contiguous(), biases.contiguous()
    out = torch.empty(need, dtype=torch.uint8, device=w.device)
    with torch.cuda.device(w.device):
        rc = lib.mfq_qmm_t_prepare(w.data_ptr(), scales.data_ptr(), biases.data_ptr(), _DTYPE_CODE[scales.dtype], N, K,
                                   group_size, bits, out.data_ptr(), torch.cuda.current_stream().cuda_stream)
    if rc != 0:
        raise _lib.MfqError("mfq_qmm_t_prepare", rc, lib.mfq_strerror(rc).decode())
    return PreparedWeights(out, scales.dtype, N, K, group_size, bits)


def quantized_matmul_prepared(x: torch.Tensor, prepared: PreparedWeights, output_dims: int | None = None,
                              bias: torch.Tensor | None = None) -> torch.Tensor:
    """``x @ dequantize(w).T (+ bias)`` on the copy ``prepare_weights`` made of
    ``w``: the second kernel of a large ``quantized_matmul`` alone, with the same
    bits in its result.  ``x``: ``[..., K]`` of the 16-bit dtype the copy was
    made in (the dtype of the scales); any number of rows, meant for some
    thousands (below that ``quantized_matmul``'s other kernels are the faster
    ones).  ``output_dims``, if given, must be the copy's.  Inference only."""
    if not isinstance(prepared, PreparedWeights):
        raise ValueError("[quantized_matmul_prepared] `prepared` must be what prepare_weights returned")
    if x.dtype != prepared.dtype:
        raise ValueError(f"[quantized_matmul_prepared] the copy holds {prepared.dtype} values, x is {x.dtype}")
    _require_hip("quantized_matmul_prepared", x, "x")
    lib = _lib.load()
    N, K = prepared.output_dims, x.shape[-1]
    if K != prepared.input_dims or (output_dims is not None and int(output_dims) != N):
        raise ValueError(f"[quantized_matmul_prepared] the prepared copy belongs to a weight of {N} x "
                         f"{prepared.input_dims}, not {output_dims if output_dims is not None else N} x {K}")
    if prepared.data.device != x.device:
        raise ValueError("[quantized_matmul_prepared] x and the prepared copy are on different devices")
    prepared = prepared.data
    lead = tuple(x.shape[:-1])
    x2 = x.reshape(-1, K).contiguous()
    M = x2.shape[0]
    y = torch.empty((M, N), dtype=x.dtype, device=x.device)
    if M == 0:
        return y.reshape(*lead, N)
    if bias is not None:
        if bias.shape != (N,):
            raise ValueError(f"[quantized_matmul_prepared] bias must have shape ({N},), got {tuple(bias.shape)}")
        bias = bias.to(x.dtype).contiguous()
    ws_bytes = lib.mfq_qmm_t_prepared_workspace_bytes(M, K, N)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device) if ws_bytes else None
    with torch.cuda.device(x.device):
        rc = lib.mfq_qmm_t_prepared(x2.data_ptr(), _DTYPE_CODE[x.dtype], M, K, prepared.data_ptr(),
                                    None if bias is None else bias.data_ptr(), N, y.data_ptr(),
                                    None if ws is None else ws.data_ptr(), ws_bytes,
                                    torch.cuda.current_stream().cuda_stream)
    if rc != 0:
        raise _lib.MfqError("mfq_qmm_t_prepared", rc, lib.mfq_strerror(rc).decode())
    return y.reshape(*lead, N)


def silu(x: torch.Tensor) -> torch.Tensor:
    """``x * sigmoid(x)`` as MLX's ``nn.silu`` evaluates it: two operations in
    ``x``'s dtype, so on a 16-bit tensor the sigmoid is rounded before the
    product is (``torch.nn.functional.silu`` rounds once)."""
    return x * torch.sigmoid(x)


def silu_quantized_matmul(x: torch.Tensor, w: torch.Tensor, scales: torch.Tensor, biases: torch.Tensor,
                          group_size: int = 64, bits: int = 4, mode: str = "affine", *,
                          bias: torch.Tensor | None = None) -> torch.Tensor:
    """``quantized_matmul(silu(x), w, scales, biases, transpose=True) (+ bias)``: the
    adaLN modulation call ``self.linear(nn.silu(text_embeddings))`` of
    src/mflux/models/flux/model/flux_transformer/ada_layer_norm_zero.py:12 (and
    ada_layer_norm_zero_single.py:12, ada_layer_norm_continuous.py:15).

    For one to four rows of 16-bit ``x`` against 4- or 8-bit weights the
    activation runs inside the matvec kernel, where the rows are converted
    anyway (``mfq_qmv_silu``); for any other call it is :func:`silu`, an elementwise
    pass, in front of :func:`quantized_matmul`.  Both round the sigmoid and the
    product to ``x``'s dtype.  Not differentiable in its fused form: with
    gradients enabled on ``x`` or ``bias`` the composed form runs.
    """
    _check_mode("quantized_matmul", mode)
    _check_group_bits("quantized_matmul", group_size, bits)
    needs_grad = torch.is_grad_enabled() and (x.requires_grad or (bias is not None and bias.requires_grad))
    K = w.shape[-1] * 32 // bits
    M = x.numel() // K if x.ndim >= 1 and x.shape[-1] == K else 0
    fusable = (1 <= M <= 4 and not needs_grad and w.ndim == 2 and bits in MATMUL_KERNEL_BITS
               and x.dtype == scales.dtype and x.dtype in (torch.bfloat16, torch.float16))
    if fusable:
        _check_packed("quantized_matmul", w, scales, biases, group_size, bits)
        _require_hip("quantized_matmul", x, "x")
        _require_hip("quantized_matmul", w, "w")
        N = w.shape[0]
        if bias is not None:
            if bias.shape != (N,):
                raise ValueError(f"[quantized_matmul] bias must have shape ({N},), got {tuple(bias.shape)}")
            bias = bias.to(x.dtype).contiguous()
        y, ok = _lib.ops().qmv_silu(x.reshape(M, K).contiguous(), w.contiguous(), scales.contiguous(),
                                    biases.contiguous(), bias, group_size, bits)
        if ok:
            return y.reshape(*x.shape[:-1], N)
    return quantized_matmul(silu(x), w, scales, biases, transpose=True, group_size=group_size, bits=bits, mode=mode,
                            bias=bias)

def layer_norm_modulate(x: torch.Tensor, scale: torch.Tensor | None = None, shift: torch.Tensor | None = None,
                        eps: float = 1e-6) -> torch.Tensor:
    """``LayerNorm(x) * (1 + scale) + shift`` over the last axis, the step in front
    of every modulated linear of the DiT blocks
    (src/mflux/models/flux/model/flux_transformer/ada_layer_norm_zero.py:22,
    joint_transformer_block.py:86-87): ``nn.LayerNorm(dims, eps, affine=False)``
    and the adaLN modulation as one pass over ``x`` instead of four.

    ``x``: ``[..., K]`` (``[B, S, K]`` in the models); ``scale``, ``shift``: ``[K]``
    or ``[B, K]`` (one vector per batch entry, broadcast over the rows of that
    entry, as ``scale[:, None]`` does in the reference), or both ``None`` for the
    plain normalisation.  Every step rounds to ``x``'s dtype as the separate
    operations do.  16-bit ``x`` on a HIP device with rows of up to 8192
    elements run in the kernel; anything else is the same sequence of torch
    operations."""
    if (scale is None) != (shift is None):
        raise ValueError("[layer_norm_modulate] scale and shift come together")
    K = x.shape[-1]
    fusable = (x.is_cuda and x.dtype in (torch.bfloat16, torch.float16) and K % 8 == 0 and K <= 8192 and x.numel() > 0
               and not (torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in (x, scale, shift))))
    vectors = None
    if scale is not None:
        if scale.shape != shift.shape or scale.shape[-1] != K or scale.numel() % K:
            raise ValueError(f"[layer_norm_modulate] scale and shift must share a shape [..., {K}], got "
                             f"{tuple(scale.shape)} and {tuple(shift.shape)}")
        vectors = scale.numel() // K
        rows = x.numel() // K
        # [B, K] against x [B, S, K]: vector b serves the S rows of entry b
        fusable = fusable and rows % vectors == 0 and (vectors == 1 or (x.ndim >= 2 and x.shape[0] == vectors)) \
            and scale.dtype == x.dtype and shift.dtype == x.dtype
    if fusable:
        y, ok = _lib.ops().layer_norm_modulate(
            x.reshape(-1, K).contiguous(),
            None if scale is None else scale.reshape(vectors, K).contiguous(),
            None if shift is None else shift.reshape(vectors, K).contiguous(), eps)
        if ok:
            return y.reshape(x.shape)
    y = torch.nn.functional.layer_norm(x, (K,), eps=eps)
    if scale is None:
        return y
    if scale.ndim == 2 and x.ndim == 3:
        scale, shift = scale[:, None, :], shift[:, None, :]
    return y * (1 + scale) + shift


EPILOGUES = {"gelu": _lib.EPILOGUE_GELU, "gate_residual": _lib.EPILOGUE_GATE_RESIDUAL, "swiglu": _lib.EPILOGUE_SWIGLU}


def gelu_approx(x: torch.Tensor) -> torch.Tensor:
    """``nn.gelu_approx`` (the tanh form) evaluated in float32 and rounded once to
    ``x``'s dtype, which is what the fused epilogue computes."""
    return torch.nn.functional.gelu(x.float(), approximate="tanh").to(x.dtype)


def swiglu_unstack(y: torch.Tensor) -> torch.Tensor:
    """``silu(g) * u`` for ``y`` whose last axis holds gate and up values in
    alternating blocks of 32 (the output of a layer made by ``nn.stack_gate_up``)."""
    blocks = y.reshape(*y.shape[:-1], y.shape[-1] // 64, 2, 32)
    return (silu(blocks[..., 0, :]) * blocks[..., 1, :]).reshape(*y.shape[:-1], y.shape[-1] // 2)


def quantized_matmul_epilogue(x: torch.Tensor, w: torch.Tensor, scales: torch.Tensor, biases: torch.Tensor, *,
                              epilogue: str, group_size: int = 64, bits: int = 4, mode: str = "affine",
                              bias: torch.Tensor | None = None, gate: torch.Tensor | None = None,
                              residual: torch.Tensor | None = None, act_from: int = 0) -> torch.Tensor:
    """A quantized linear and what the reference does to its output next, as one
    kernel where a GEMM kernel runs (more than 16 rows of 16-bit ``x``); any other
    call runs :func:`quantized_matmul` and the same operations on its result.

    ``epilogue``:
      ``"gelu"``           ``gelu_approx(linear(x))`` on the columns from ``act_from``
                           (a multiple of 8) on: ``nn.gelu_approx(self.proj_mlp(.))``,
                           src/mflux/models/flux/model/flux_transformer/single_transformer_block.py:53-54;
      ``"gate_residual"``  ``residual + gate * linear(x)`` with ``gate`` of shape
                           ``[N]`` (or ``[1, N]``) and ``residual`` of the output's
                           shape: single_transformer_block.py:45,57,
                           joint_transformer_block.py:84-90;
      ``"swiglu"``         ``silu(g) * u`` for a weight whose rows alternate between
                           the gate and the up projection in blocks of 32
                           (``nn.stack_gate_up``); the result has ``N / 2`` columns:
                           src/mflux/models/z_image/model/z_image_transformer/feed_forward.py:13.
    Every step rounds to ``x``'s dtype as the separate operations do.  Inference
    only (no autograd through the fused form: with gradients enabled on an input
    the composed form runs)."""
    _check_mode("quantized_matmul", mode)
    _check_group_bits("quantized_matmul", group_size, bits)
    if epilogue not in EPILOGUES:
        raise ValueError(f"[quantized_matmul] unknown epilogue '{epilogue}' (one of {sorted(EPILOGUES)})")
    _check_packed("quantized_matmul", w, scales, biases, group_size, bits)
    N = w.shape[0]
    K = w.shape[-1] * 32 // bits
    if epilogue == "gate_residual":
        if gate is None or residual is None:
            raise ValueError("[quantized_matmul] the gate_residual epilogue needs gate and residual")
        if gate.numel() != N or tuple(residual.shape) != (*x.shape[:-1], N):
            raise ValueError(f"[quantized_matmul] gate must hold {N} values and residual have shape "
                             f"{(*x.shape[:-1], N)}; got {tuple(gate.shape)} and {tuple(residual.shape)}")
    if epilogue == "swiglu" and N % 64:
        raise ValueError(f"[quantized_matmul] the swiglu epilogue needs gate and up rows in blocks of 32 (N % 64 == 0), got N = {N}")
    if epilogue == "gelu" and (act_from < 0 or act_from > N or act_from % 8):
        raise ValueError(f"[quantized_matmul] act_from must be a multiple of 8 in [0, {N}], got {act_from}")
    tensors = [t for t in (x, bias, gate, residual) if t is not None]
    needs_grad = torch.is_grad_enabled() and any(t.requires_grad for t in tensors)
    M = x.numel() // K if x.ndim >= 1 and x.shape[-1] == K else 0
    fusable = (M > 16 and not needs_grad and w.ndim == 2 and x.dtype == scales.dtype
               and x.dtype in (torch.bfloat16, torch.float16)
               and all(t.dtype == x.dtype for t in tensors))
    if fusable:
        _require_hip("quantized_matmul", x, "x")
        _require_hip("quantized_matmul", w, "w")
        if bias is not None and bias.shape != (N,):
            raise ValueError(f"[quantized_matmul] bias must have shape ({N},), got {tuple(bias.shape)}")
        y, ok = _lib.ops().qmm_t_epilogue(
            x.reshape(M, K).contiguous(), w.contiguous(), scales.contiguous(), biases.contiguous(),
            None if bias is None else bias.contiguous(), group_size, bits, EPILOGUES[epilogue],
            None if gate is None else gate.reshape(N).contiguous(),
            None if residual is None else residual.reshape(M, N).contiguous(), act_from)
        if ok:
            return y.reshape(*x.shape[:-1], y.shape[-1])
    y = quantized_matmul(x, w, scales, biases, transpose=True, group_size=group_size, bits=bits, mode=mode, bias=bias)
    if epilogue == "gelu":
        if act_from == 0:
            return gelu_approx(y)
        return torch.cat([y[..., :act_from], gelu_approx(y[..., act_from:])], dim=-1)
    if epilogue == "gate_residual":
        return residual + gate.reshape(N) * y
    return swiglu_unstack(y)


def _low_rank_operands(low_rank, lead: tuple, M: int, N: int, compute: torch.dtype):
    """Checks ``(t, bs)`` against the product's shape; returns them as contiguous
    ``[M, R]`` / ``[N, R]`` matrices in the compute dtype."""
    t, bs = low_rank
    if t.ndim < 1 or tuple(t.shape[:-1]) != lead or bs.ndim != 2 or bs.shape[0] != N or bs.shape[1] != t.shape[-1]:
        raise ValueError(f"[quantized_matmul] low_rank must be (t [..., R], bs [{N}, R]) with t's leading "
                         f"dimensions {lead}; got {tuple(t.shape)} and {tuple(bs.shape)}")
    R = bs.shape[1]
    if R == 0 or R % 16 or R > 1024:
        raise ValueError(f"[quantized_matmul] the low rank must be a multiple of 16 up to 1024 (pad with zeros), got {R}")
    _require_hip("quantized_matmul", t, "low_rank t")
    _require_hip("quantized_matmul", bs, "low_rank bs")
    return t.reshape(M, R).to(compute).contiguous(), bs.to(compute).contiguous(), R


def _quantized_matmul_forward(x: torch.Tensor, w: torch.Tensor, scales: torch.Tensor, biases: torch.Tensor,
                              group_size: int, bits: int, bias: torch.Tensor | None,
                              low_rank: tuple[torch.Tensor, torch.Tensor] | None = None) -> torch.Tensor:
    """``x @ dequantize(w).T`` with float32 accumulation.

    ``low_rank = (t, bs)`` (not part of ``mx.quantized_matmul``) adds
    ``t @ bs.T`` to the product: the LoRA branch of
    src/mflux/models/common/lora/layer/linear_lora_layer.py:50-53 with
    ``t = x @ lora_A`` (``[..., R]``) and ``bs = scale * lora_B.T`` (``[N, R]``),
    several adapters concatenated along ``R``, ``R`` zero-padded to a multiple
    of 16.  The GEMM kernels (more than 16 rows) accumulate it with the product
    before the one rounding; the matvec kernels are followed by a small second
    kernel.

    ``x``: ``[..., K]``; ``w``: packed ``[N, K*bits/32]``.  The result has dtype
    ``result_type(x, scales)``; when that is float32 (float32 ``x`` against
    16-bit scales) ``x`` is rounded to the dtype of ``scales`` for the matrix
    cores and only the accumulation and output are float32.  ``bias`` (not part
    of ``mx.quantized_matmul``) fuses the add of ``QuantizedLinear`` into the
    kernel's epilogue with the same two roundings as a separate add.
    """
    _check_packed("quantized_matmul", w, scales, biases, group_size, bits)
    if w.ndim != 2:
        raise NotImplementedError("[quantized_matmul] batched weights are not implemented in this build")
    if x.dtype not in _DTYPE_CODE:
        raise ValueError(f"[quantized_matmul] Only real floating types are supported but {x.dtype} was provided "
                         "for the input")
    if scales.dtype == torch.float32:
        raise NotImplementedError("[quantized_matmul] float32 scales are not implemented in this build")
    N = w.shape[0]
    K = w.shape[1] * 32 // bits
    if x.ndim < 1 or x.shape[-1] != K:
        raise ValueError(
            f"[quantized_matmul] Last dimension of first input with shape {tuple(x.shape)} does not match the "
            f"expanded quantized matrix ({K}, {N}) computed from shape {tuple(w.shape)} with "
            f"group_size={group_size}, bits={bits} and transpose=true"
        )
    _require_hip("quantized_matmul", x, "x")
    _require_hip("quantized_matmul", w, "w")
    out_dtype = torch.result_type(x, scales)
    compute = scales.dtype
    lead = tuple(x.shape[:-1])
    x2 = x.reshape(-1, K)
    if x2.dtype != compute:
        x2 = x2.to(compute)
    x2 = x2.contiguous()
    M = x2.shape[0]
    if M == 0:
        return torch.empty((*lead, N), dtype=out_dtype, device=x.device)
    if bias is not None:
        if bias.shape != (N,):
            raise ValueError(f"[quantized_matmul] bias must have shape ({N},), got {tuple(bias.shape)}")
        bias = bias.to(compute).contiguous()
    w, scales, biases = w.contiguous(), scales.contiguous(), biases.contiguous()
    ops = _lib.ops()
    lr_t = lr_bs = None
    if low_rank is not None:
        lr_t, lr_bs, _ = _low_rank_operands(low_rank, lead, M, N, compute)
    y, ok = ops.qmm_t(x2, w, scales, biases, bias, group_size, bits, out_dtype, lr_t, lr_bs)
    if not ok:
        raise NotImplementedError(f"[quantized_matmul] no kernel for x {tuple(x.shape)} against a weight of "
                                  f"{N} x {K} (an operand exceeds 2 GiB: split the rows of x)")
    return y.reshape(*lead, N)
