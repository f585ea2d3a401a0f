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

    def forward(self, x: torch.Tensor) -> torch.Tensor:
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
