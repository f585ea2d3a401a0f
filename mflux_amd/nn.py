"""Module-level API: ``quantize``, ``QuantizedLinear``, ``Linear``,
``QuantizedEmbedding``, ``Embedding``.

Mirrors the part of ``mlx.nn`` that mflux uses to quantize a model and to run
it: ``nn.quantize(model, class_predicate=..., bits=...)`` at
src/mflux/models/common/weights/loading/weight_applier.py:43,46,103, the
``hasattr(module, "to_quantized")`` predicates
(src/mflux/models/flux/weights/flux_weight_definition.py:79-81) and the
attributes the LoRA wrappers read from a quantized layer
(src/mflux/models/common/lora/layer/linear_lora_layer.py:14-16:
``weight.shape == (N, K*bits/32)`` and ``bits``).
"""
from __future__ import annotations

import contextlib
import math
import weakref
from typing import Callable

import torch

from . import core


def _defaults(group_size: int | None, bits: int | None) -> tuple[int, int]:
    return (64 if group_size is None else group_size, 4 if bits is None else bits)


_PLACEHOLDERS = False


@contextlib.contextmanager
def placeholder_quantization():
    """Inside this context ``to_quantized`` / ``from_linear`` build quantized
    layers of the right shapes and dtypes with zeroed tensors instead of
    running the quantize kernel.  For loading stored codes: the reference
    quantizes the freshly initialised model and then overwrites every packed
    tensor (src/mflux/models/common/weights/loading/weight_applier.py:45-47);
    quantizing values that are about to be replaced is skipped here."""
    global _PLACEHOLDERS
    previous, _PLACEHOLDERS = _PLACEHOLDERS, True
    try:
        yield
    finally:
        _PLACEHOLDERS = previous


class QuantizedLinear(torch.nn.Module):
    """``y = quantized_matmul(x, weight, scales, biases) (+ bias)``.

    Tensors are named as MLX names them (``weight`` packed uint32
    ``[N, K*bits/32]``, ``scales``/``biases`` ``[N, K/group_size]``, optional
    ``bias`` ``[N]``) and are frozen (buffers, no gradient), so
    ``state_dict()`` is exactly what mflux saves for the layer.
    """

    def __init__(self, input_dims: int, output_dims: int, bias: bool = True, group_size: int | None = None,
                 bits: int | None = None, mode: str = "affine", *, device=None, dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        self.group_size, self.bits = _defaults(group_size, bits)
        self.mode = mode
        core._check_mode("QuantizedLinear", mode)
        core._check_group_bits("QuantizedLinear", self.group_size, self.bits)
        if input_dims % self.group_size:
            raise ValueError(
                "[quantize] The last dimension of the matrix needs to be divisible by the quantization "
                f"group size {self.group_size}. However the provided matrix has shape {(output_dims, input_dims)}"
            )
        device = torch.device("cpu" if device is None else device)
        if device.type == "cuda":
            bound = math.sqrt(1.0 / input_dims)
            w = torch.empty((output_dims, input_dims), device=device, dtype=torch.float32).uniform_(-bound, bound)
            wq, scales, biases = core.quantize(w.to(dtype), self.group_size, self.bits)
        else:  # placeholders of the right shape, to be filled by load_state_dict / update
            wq = torch.zeros((output_dims, input_dims * self.bits // 32), dtype=torch.uint32, device=device)
            scales = torch.zeros((output_dims, input_dims // self.group_size), dtype=dtype, device=device)
            biases = torch.zeros_like(scales)
        self.register_buffer("weight", wq)
        self.register_buffer("scales", scales)
        self.register_buffer("biases", biases)
        if bias:
            self.register_buffer("bias", torch.zeros((output_dims,), dtype=dtype, device=device))
        else:
            self.bias = None

    @property
    def input_dims(self) -> int:
        return self.weight.shape[1] * 32 // self.bits

    @property
    def output_dims(self) -> int:
        return self.weight.shape[0]

    def extra_repr(self) -> str:
        return (f"input_dims={self.input_dims}, output_dims={self.output_dims}, bias={self.bias is not None}, "
                f"group_size={self.group_size}, bits={self.bits}, mode={self.mode}")

    PREPARED_MIN_ROWS = 2048  # from here on forward() multiplies with the prepared copy, if there is one

    def _weights_key(self):
        # weak references, not addresses: a fresh tensor can reuse a freed tensor's address at version 0
        return tuple((weakref.ref(t), t._version) for t in (self.weight, self.scales, self.biases))

    def _prepared_is_current(self) -> bool:
        key = getattr(self, "_prepared_key", None)
        now = (self.weight, self.scales, self.biases)
        return key is not None and all(ref() is t and version == t._version for (ref, version), t in zip(key, now))

    def _apply(self, fn, *args, **kwargs):
        # .to() / .cuda() / .half(): the kept copy belongs to the old tensors
        self._prepared = None
        self._prepared_key = None
        return super()._apply(fn, *args, **kwargs)

    def prepare(self) -> bool:
        """Keeps a 16-bit copy of the dequantised weights in the order the large-M
        GEMM consumes them (``core.prepare_weights``: 2 bytes per weight of device
        memory), so that calls with thousands of rows skip the dequantisation
        pass.  Not part of MLX's layer.  The copy is not part of ``state_dict()``
        and is made again when the layer's tensors have been replaced or written
        to.  Returns False (and keeps nothing) where the library has no such copy
        for the layer's shape."""
        self._prepared = core.prepare_weights(self.weight, self.scales, self.biases, self.group_size, self.bits)
        self._prepared_key = self._weights_key() if self._prepared is not None else None
        return self._prepared is not None

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if (getattr(self, "_prepared", None) is not None and x.dtype == self.scales.dtype and x.shape[-1] > 0
                and x.numel() // x.shape[-1] >= self.PREPARED_MIN_ROWS and not (torch.is_grad_enabled() and x.requires_grad)):
            if not self._prepared_is_current():
                self.prepare()
            if self._prepared is not None:
                return core.quantized_matmul_prepared(x, self._prepared, self.output_dims, self.bias)
        return core.quantized_matmul(x, self.weight, self.scales, self.biases, transpose=True,
                                     group_size=self.group_size, bits=self.bits, mode=self.mode, bias=self.bias)

    def silu_forward(self, x: torch.Tensor) -> torch.Tensor:
        """``self(silu(x))``, the activation inside the matvec kernel when ``x`` is one row."""
        return core.silu_quantized_matmul(x, self.weight, self.scales, self.biases, group_size=self.group_size,
                                          bits=self.bits, mode=self.mode, bias=self.bias)

    @classmethod
    def from_linear(cls, linear_layer: torch.nn.Module, group_size: int | None = None, bits: int | None = None,
                    mode: str = "affine") -> "QuantizedLinear":
        weight = linear_layer.weight.detach()
        output_dims, input_dims = weight.shape
        group_size, bits = _defaults(group_size, bits)
        ql = cls.__new__(cls)
        torch.nn.Module.__init__(ql)
        ql.group_size, ql.bits, ql.mode = group_size, bits, mode
        if _PLACEHOLDERS:
            core._check_mode("quantize", mode)
            core._check_group_bits("quantize", group_size, bits)
            if input_dims % group_size:
                raise ValueError(
                    "[quantize] The last dimension of the matrix needs to be divisible by the quantization "
                    f"group size {group_size}. However the provided matrix has shape {tuple(weight.shape)}"
                )
            wq = torch.zeros((output_dims, input_dims * bits // 32), dtype=torch.uint32, device=weight.device)
            scales = torch.zeros((output_dims, input_dims // group_size), dtype=weight.dtype, device=weight.device)
            biases = torch.zeros_like(scales)
        else:
            wq, scales, biases = core.quantize(weight, group_size, bits, mode)
        ql.register_buffer("weight", wq)
        ql.register_buffer("scales", scales)
        ql.register_buffer("biases", biases)
        lin_bias = getattr(linear_layer, "bias", None)
        if lin_bias is not None:
            ql.register_buffer("bias", lin_bias.detach())
        else:
            ql.bias = None
        return ql


def silu(x: torch.Tensor) -> torch.Tensor:
    """MLX's ``nn.silu``: ``x * sigmoid(x)`` as two operations in ``x``'s dtype."""
    return core.silu(x)


def silu_linear(layer: torch.nn.Module, x: torch.Tensor) -> torch.Tensor:
    """``layer(nn.silu(x))``, the adaLN modulation call of
    src/mflux/models/flux/model/flux_transformer/ada_layer_norm_zero.py:12, as
    one kernel when ``layer`` is a :class:`QuantizedLinear` and ``x`` one row;
    the composition otherwise (float linears, LoRA wrappers, more rows)."""
    if type(layer) is QuantizedLinear:
        return layer.silu_forward(x)
    return layer(core.silu(x))


def _linear_parts(layer: torch.nn.Module, fn: str):
    if not isinstance(layer, QuantizedLinear):
        raise ValueError(f"[{fn}] expected a QuantizedLinear, got {type(layer).__name__}")
    return layer.weight, layer.scales, layer.biases


def layer_norm_modulate(x: torch.Tensor, scale: torch.Tensor | None = None, shift: torch.Tensor | None = None,
                        eps: float = 1e-6) -> torch.Tensor:
    """``nn.LayerNorm(dims, eps, affine=False)(x) * (1 + scale) + shift`` as one
    pass (``core.layer_norm_modulate``): the step in front of the modulated
    linears, e.g. src/mflux/models/flux/model/flux_transformer/ada_layer_norm_zero.py:22."""
    return core.layer_norm_modulate(x, scale, shift, eps)


def gelu_linear(layer: torch.nn.Module, x: torch.Tensor, act_from: int = 0) -> torch.Tensor:
    """``nn.gelu_approx(layer(x))`` as one kernel: the activation behind
    ``proj_mlp`` of a single-stream block
    (src/mflux/models/flux/model/flux_transformer/single_transformer_block.py:53-54)
    and between the feed-forward linears of a joint block.  ``act_from``: the
    first output column the activation applies to, for a layer that stacks q, k,
    v and proj_mlp (``concat_quantized``) and activates only the last part.  A
    float layer gets the composed form."""
    if not isinstance(layer, QuantizedLinear):
        y = layer(x)
        return torch.cat([y[..., :act_from], core.gelu_approx(y[..., act_from:])], dim=-1) if act_from else core.gelu_approx(y)
    w, s, b = _linear_parts(layer, "gelu_linear")
    return core.quantized_matmul_epilogue(x, w, s, b, epilogue="gelu", group_size=layer.group_size, bits=layer.bits,
                                          mode=layer.mode, bias=layer.bias, act_from=act_from)


def gate_residual_linear(layer: torch.nn.Module, x: torch.Tensor, gate: torch.Tensor,
                         residual: torch.Tensor) -> torch.Tensor:
    """``residual + gate * layer(x)`` as one kernel, ``gate`` one value per output
    feature (``[N]`` or ``[1, N]``): ``residual + gate * proj_out(.)`` of a
    single-stream block (single_transformer_block.py:45,57) and ``hidden + gate *
    ff(.)`` / ``hidden + gate * attn_output`` of a joint block
    (joint_transformer_block.py:84-90).  The reference's gate is one vector per
    batch entry, expanded over the sequence (``mx.expand_dims(gate, 1)``): a
    ``gate`` of shape ``[B, N]`` or ``[B, 1, N]`` next to ``x`` of ``[B, S, K]``
    runs the kernel once per batch entry, each with its own vector.  A float
    layer gets the composed form."""
    N = layer.output_dims if isinstance(layer, QuantizedLinear) else layer.weight.shape[0]
    if gate.numel() != N:
        B = x.shape[0] if x.ndim >= 3 else 0
        if B and gate.numel() == B * N and tuple(gate.shape) in ((B, N), (B, 1, N)) and residual.shape[0] == B:
            gates = gate.reshape(B, N)
            return torch.stack([gate_residual_linear(layer, x[i], gates[i], residual[i]) for i in range(B)])
        raise ValueError(f"[gate_residual_linear] gate must hold {N} values, or {N} per batch entry as [B, {N}] or "
                         f"[B, 1, {N}] next to x of [B, S, K]; got {tuple(gate.shape)} for x of {tuple(x.shape)}")
    if not isinstance(layer, QuantizedLinear):
        return residual + gate.reshape(-1) * layer(x)
    w, s, b = _linear_parts(layer, "gate_residual_linear")
    return core.quantized_matmul_epilogue(x, w, s, b, epilogue="gate_residual", group_size=layer.group_size,
                                          bits=layer.bits, mode=layer.mode, bias=layer.bias, gate=gate,
                                          residual=residual)


def stack_gate_up(gate_layer: QuantizedLinear, up_layer: QuantizedLinear) -> QuantizedLinear:
    """The gate (``w1``) and up (``w3``) projections of a SwiGLU feed-forward
    (src/mflux/models/z_image/model/z_image_transformer/feed_forward.py:8-13) as
    one ``QuantizedLinear`` whose rows alternate between the two in blocks of 32:
    rows ``64 i .. 64 i + 31`` are rows ``32 i ..`` of the gate projection, the next
    32 the same rows of the up projection.  A packed row belongs to its output
    feature alone, so this is a permutation of rows of codes, scales and biases
    and needs no requantization.  ``swiglu_linear`` evaluates ``silu(w1 x) * w3 x``
    on it in one kernel: both values of an output land in the same register of
    the same lane."""
    for layer in (gate_layer, up_layer):
        _linear_parts(layer, "stack_gate_up")
    a, b = gate_layer, up_layer
    if (a.input_dims, a.output_dims, a.group_size, a.bits, a.mode, a.scales.dtype) != (
            b.input_dims, b.output_dims, b.group_size, b.bits, b.mode, b.scales.dtype):
        raise ValueError("[stack_gate_up] the two layers must share shape, group_size, bits, mode and dtype")
    if a.output_dims % 32:
        raise ValueError(f"[stack_gate_up] output_dims must be a multiple of 32, got {a.output_dims}")
    if (a.bias is None) != (b.bias is None):
        raise ValueError("[stack_gate_up] both layers or neither must have a bias")

    def weave(p, q):
        return torch.stack([p.reshape(-1, 32, *p.shape[1:]), q.reshape(-1, 32, *q.shape[1:])], dim=1).reshape(
            2 * p.shape[0], *p.shape[1:])

    out = QuantizedLinear.__new__(QuantizedLinear)
    torch.nn.Module.__init__(out)
    out.group_size, out.bits, out.mode = a.group_size, a.bits, a.mode
    out.register_buffer("weight", weave(a.weight.view(torch.int32), b.weight.view(torch.int32)).view(torch.uint32))
    out.register_buffer("scales", weave(a.scales, b.scales))
    out.register_buffer("biases", weave(a.biases, b.biases))
    if a.bias is not None:
        out.register_buffer("bias", weave(a.bias, b.bias))
    else:
        out.bias = None
    return out


def swiglu_linear(stacked: QuantizedLinear, x: torch.Tensor) -> torch.Tensor:
    """``silu(w1 x) * w3 x`` for ``stacked = stack_gate_up(w1, w3)``: one GEMM over
    both projections whose epilogue writes the ``[..., N / 2]`` product, instead
    of two GEMMs and three element-wise passes."""
    w, s, b = _linear_parts(stacked, "swiglu_linear")
    return core.quantized_matmul_epilogue(x, w, s, b, epilogue="swiglu", group_size=stacked.group_size,
                                          bits=stacked.bits, mode=stacked.mode, bias=stacked.bias)


def concat_quantized(layers: list[QuantizedLinear], share_storage: bool = False) -> QuantizedLinear:
    """One ``QuantizedLinear`` whose output is the outputs of ``layers`` side by
    side: the packed rows, scales and biases of a weight belong to its output
    feature alone, so stacking them along N needs no requantization.  The q, k
    and v projections of an attention block (e.g.
    src/mflux/models/flux/model/flux_transformer/common/attention_utils.py:21-23,
    three calls on the same input) become one launch over three times the
    tiles, which fills the GPU better than three small ones; the caller splits
    the result with ``split`` / slicing (views, no copy).  The inputs are left
    untouched (their tensors are copied) unless ``share_storage`` is set: then
    every input layer's tensors become views of the stacked ones, so the stack
    costs no memory and the layers keep working on their own.  The views stay
    in step with the stack as long as new values are written INTO the layers'
    tensors: ``weights.update_module`` and ``lora.bake_and_strip_lora`` copy in
    place when shape and dtype are unchanged; assigning a fresh tensor to
    ``layer.weight`` detaches that layer from the stack, so stack after loading.

    The same serves the adaLN modulation linears of a whole model
    (src/mflux/models/flux/model/flux_transformer/ada_layer_norm_zero.py:12 in
    every block): all of them take the same ``silu(text_embeddings)``, so
    ``silu_linear(concat_quantized(all_of_them, share_storage=True), temb)`` at
    the start of a step is one matvec over gigabytes of weights instead of one
    launch of 30 to 60 MB per block, each of which pays the launch's fixed cost."""
    if not layers:
        raise ValueError("[concat_quantized] needs at least one layer")
    first = layers[0]
    for layer in layers:
        if not isinstance(layer, QuantizedLinear):
            raise ValueError(f"[concat_quantized] expected QuantizedLinear layers, got {type(layer).__name__}")
        if (layer.input_dims, layer.group_size, layer.bits, layer.mode, layer.scales.dtype) != (
                first.input_dims, first.group_size, first.bits, first.mode, first.scales.dtype):
            raise ValueError("[concat_quantized] the layers must share input_dims, group_size, bits, mode and dtype")
    out = QuantizedLinear.__new__(QuantizedLinear)
    torch.nn.Module.__init__(out)
    out.group_size, out.bits, out.mode = first.group_size, first.bits, first.mode
    out.register_buffer("weight", torch.cat([layer.weight for layer in layers], dim=0))
    out.register_buffer("scales", torch.cat([layer.scales for layer in layers], dim=0))
    out.register_buffer("biases", torch.cat([layer.biases for layer in layers], dim=0))
    if any(layer.bias is not None for layer in layers):
        parts = [layer.bias if layer.bias is not None else
                 torch.zeros(layer.output_dims, dtype=first.scales.dtype, device=first.scales.device)
                 for layer in layers]
        out.register_buffer("bias", torch.cat(parts, dim=0))
    else:
        out.bias = None
    if share_storage:
        row = 0
        for layer in layers:
            end = row + layer.output_dims
            layer._buffers["weight"] = out.weight[row:end]
            layer._buffers["scales"] = out.scales[row:end]
            layer._buffers["biases"] = out.biases[row:end]
            if layer.bias is not None:
                layer._buffers["bias"] = out.bias[row:end]
            row = end
    return out


def prepare(model: torch.nn.Module, min_output_dims: int = 0) -> int:
    """Calls ``QuantizedLinear.prepare()`` on every quantized linear of ``model``
    with at least ``min_output_dims`` output features (after loading, baking
    and stacking: the copy follows later changes to a layer's tensors, at the
    price of making it again).  Not part of MLX.  Returns the bytes of device
    memory the kept copies take: 2 per weight, 24 GB for FLUX.1's transformer."""
    held = 0
    for module in model.modules():
        if isinstance(module, QuantizedLinear) and module.output_dims >= min_output_dims and module.prepare():
            held += module._prepared.numel()
    return held


class Linear(torch.nn.Linear):
    """``torch.nn.Linear`` with MLX's ``to_quantized`` hook, so that the
    reference's ``hasattr(module, "to_quantized")`` predicates select it."""

    def to_quantized(self, group_size: int | None = None, bits: int | None = None, mode: str = "affine"):
        return QuantizedLinear.from_linear(self, group_size, bits, mode)


class QuantizedEmbedding(torch.nn.Module):
    """Embedding table held as packed codes: ``forward(ids)`` gathers and
    dequantizes the rows, ``as_linear(x)`` multiplies by the transposed table.

    What MLX's ``nn.Embedding.to_quantized`` produces, and therefore what
    ``nn.quantize`` with the default predicate turns every embedding into
    (e.g. src/mflux/models/flux/model/flux_text_encoder/t5_encoder/t5_encoder.py:11).
    """

    def __init__(self, num_embeddings: int, dims: int, group_size: int | None = None, bits: int | None = None,
                 mode: str = "affine", *, device=None, dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        self.group_size, self.bits = _defaults(group_size, bits)
        self.mode = mode
        self.num_embeddings, self.dims = num_embeddings, dims
        core._check_mode("QuantizedEmbedding", mode)
        core._check_group_bits("QuantizedEmbedding", self.group_size, self.bits)
        if dims % self.group_size:
            raise ValueError(
                "[quantize] The last dimension of the matrix needs to be divisible by the quantization "
                f"group size {self.group_size}. However the provided matrix has shape {(num_embeddings, dims)}"
            )
        device = torch.device("cpu" if device is None else device)
        if device.type == "cuda":
            w = torch.randn((num_embeddings, dims), device=device, dtype=torch.float32) * math.sqrt(1.0 / dims)
            wq, scales, biases = core.quantize(w.to(dtype), self.group_size, self.bits)
        else:
            wq = torch.zeros((num_embeddings, dims * self.bits // 32), dtype=torch.uint32, device=device)
            scales = torch.zeros((num_embeddings, dims // self.group_size), dtype=dtype, device=device)
            biases = torch.zeros_like(scales)
        self.register_buffer("weight", wq)
        self.register_buffer("scales", scales)
        self.register_buffer("biases", biases)

    def extra_repr(self) -> str:
        return f"{self.num_embeddings}, {self.dims}, group_size={self.group_size}, bits={self.bits}, mode={self.mode}"

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return core.dequantize_rows(self.weight, self.scales, self.biases, x, group_size=self.group_size,
                                    bits=self.bits, mode=self.mode)

    def as_linear(self, x: torch.Tensor) -> torch.Tensor:
        return core.quantized_matmul(x, self.weight, self.scales, self.biases, transpose=True,
                                     group_size=self.group_size, bits=self.bits, mode=self.mode)

    @classmethod
    def from_embedding(cls, embedding_layer: torch.nn.Module, group_size: int | None = None, bits: int | None = None,
                       mode: str = "affine") -> "QuantizedEmbedding":
        weight = embedding_layer.weight.detach()
        num_embeddings, dims = weight.shape
        group_size, bits = _defaults(group_size, bits)
        qe = cls.__new__(cls)
        torch.nn.Module.__init__(qe)
        qe.group_size, qe.bits, qe.mode = group_size, bits, mode
        qe.num_embeddings, qe.dims = num_embeddings, dims
        if _PLACEHOLDERS:
            core._check_mode("quantize", mode)
            core._check_group_bits("quantize", group_size, bits)
            if dims % group_size:
                raise ValueError(
                    "[quantize] The last dimension of the matrix needs to be divisible by the quantization "
                    f"group size {group_size}. However the provided matrix has shape {tuple(weight.shape)}"
                )
            wq = torch.zeros((num_embeddings, dims * bits // 32), dtype=torch.uint32, device=weight.device)
            scales = torch.zeros((num_embeddings, dims // group_size), dtype=weight.dtype, device=weight.device)
            biases = torch.zeros_like(scales)
        else:
            wq, scales, biases = core.quantize(weight, group_size, bits, mode)
        qe.register_buffer("weight", wq)
        qe.register_buffer("scales", scales)
        qe.register_buffer("biases", biases)
        return qe


class Embedding(torch.nn.Embedding):
    """``torch.nn.Embedding`` with MLX's ``to_quantized`` and ``as_linear``."""

    def as_linear(self, x: torch.Tensor) -> torch.Tensor:
        return torch.nn.functional.linear(x, self.weight)

    def to_quantized(self, group_size: int | None = None, bits: int | None = None, mode: str = "affine"):
        return QuantizedEmbedding.from_embedding(self, group_size, bits, mode)


def leaf_modules(model: torch.nn.Module):
    """(dotted path, parent, attribute name, module) of every module without
    children, in registration order -- MLX's ``Module.leaf_modules()`` with the
    same path spelling (``blocks.0.attn.to_q``)."""
    out = []
    for path, module in model.named_modules():
        if path == "" or any(True for _ in module.children()):
            continue
        parent_path, _, name = path.rpartition(".")
        parent = model.get_submodule(parent_path) if parent_path else model
        out.append((path, parent, name, module))
    return out


def quantize(model: torch.nn.Module, group_size: int | None = None, bits: int | None = None, *,
             mode: str = "affine", class_predicate: Callable | None = None) -> torch.nn.Module:
    """Replaces, in place, every leaf module the predicate selects by its
    quantized counterpart (``module.to_quantized(...)``).

    ``class_predicate(path, module)`` returns a bool, or a dict of keyword
    arguments for ``to_quantized``.  The default selects every module that has a
    ``to_quantized`` method.  A truthy answer for a module without one raises
    ``ValueError``.  Returns the model.
    """
    group_size, bits = _defaults(group_size, bits)
    class_predicate = class_predicate or (lambda _, m: hasattr(m, "to_quantized"))
    for path, parent, name, module in leaf_modules(model):
        answer = class_predicate(path, module)
        if not answer:
            continue
        if not hasattr(module, "to_quantized"):
            raise ValueError(f"Unable to quantize model of type {type(module)}")
        if isinstance(answer, bool):
            kwargs = {"group_size": group_size, "bits": bits, "mode": mode}
        elif isinstance(answer, dict):
            kwargs = answer
        else:
            raise ValueError("``class_predicate`` must return a bool or a dict of parameters to pass to "
                             "``to_quantized``")
        parent._modules[name] = module.to_quantized(**kwargs)
    return model
