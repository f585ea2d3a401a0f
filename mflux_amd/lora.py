"""LoRA adapters on (quantized) linear layers.

Mirrors mflux's wrappers, same names and attributes:
``LoRALinear`` (src/mflux/models/common/lora/layer/linear_lora_layer.py:8-53:
``from_linear(linear, r, scale)``, ``linear``, ``scale``, ``lora_A [K, r]``,
``lora_B [r, N]``, ``base + scale * (x @ A) @ B``) and ``FusedLoRALinear``
(src/mflux/models/common/lora/layer/fused_linear_lora_layer.py:7-20:
``base_linear``, ``loras``, the sum over the adapters).

Around a ``QuantizedLinear`` base on the GPU, at inference, the whole layer is
one call of the quantized matmul: the adapters' down-projections are
concatenated into one ``[K, R]`` matrix (one small library GEMM gives ``t = x @ A``),
the scaled up-projections into one ``[N, R]`` matrix, and the kernel treats
them as ``R`` more ``k`` of the same product.  When gradients are needed, or
the base is not quantized, the layer is the reference's composition of
separate matmuls.
"""
from __future__ import annotations

import math

import torch

from . import _lib, core
from .nn import Linear, QuantizedLinear

_RANK_STEP = 16  # the kernels take the low rank in steps of 16


class LoRALinear(torch.nn.Module):
    @staticmethod
    def from_linear(linear: torch.nn.Module, r: int = 16, scale: float = 1.0) -> "LoRALinear":
        output_dims, input_dims = linear.weight.shape
        if isinstance(linear, QuantizedLinear):
            # packed words -> elements (the reference multiplies by 32 // bits, which is only right for 4 and 8 bits)
            input_dims = input_dims * 32 // linear.bits
        ref = linear.scales if isinstance(linear, QuantizedLinear) else linear.weight
        lora_lin = LoRALinear(input_dims=input_dims, output_dims=output_dims, r=r, scale=scale, device=ref.device,
                              dtype=ref.dtype, _make_linear=False)
        lora_lin.linear = linear
        return lora_lin

    def __init__(self, input_dims: int, output_dims: int, r: int = 8, scale: float = 1.0, bias: bool = False, *,
                 device=None, dtype: torch.dtype = torch.bfloat16, _make_linear: bool = True):
        super().__init__()
        if _make_linear:
            self.linear = Linear(input_dims, output_dims, bias=bias, device=device, dtype=dtype)
        self.scale = scale
        bound = 1 / math.sqrt(input_dims)
        make = lambda *shape: torch.nn.Parameter(
            torch.empty(shape, device=device, dtype=torch.float32).uniform_(-bound, bound).to(dtype))
        self.lora_A = make(input_dims, r)
        self.lora_B = make(r, output_dims)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return _forward(self, self.linear, [self], x)


class FusedLoRALinear(torch.nn.Module):
    def __init__(self, base_linear: torch.nn.Module, loras: list[LoRALinear]):
        super().__init__()
        self.base_linear = base_linear
        self.loras = torch.nn.ModuleList(loras)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return _forward(self, self.base_linear, list(self.loras), x)


def _composed(base: torch.nn.Module, loras: list[LoRALinear], x: torch.Tensor) -> torch.Tensor:
    """The reference's arithmetic: separate matmuls, every intermediate rounded."""
    out = base(x)
    if len(loras) == 1:
        lora = loras[0]
        return out + lora.scale * torch.matmul(torch.matmul(x.to(lora.lora_A.dtype), lora.lora_A), lora.lora_B)
    lora_out = torch.zeros_like(out)
    for lora in loras:
        lora_out = lora_out + lora.scale * torch.matmul(torch.matmul(x.to(lora.lora_A.dtype), lora.lora_A),
                                                        lora.lora_B)
    return out + lora_out


def pack_adapters(loras: list[LoRALinear], dtype: torch.dtype) -> tuple[torch.Tensor, torch.Tensor]:
    """``(a_cat [K, R], bs [N, R])`` for ``quantized_matmul(..., low_rank=(x @ a_cat, bs))``:
    the down-projections side by side and the up-projections, scaled in float32
    and transposed, side by side, ``R`` = the sum of the ranks rounded up to a
    multiple of 16 with zero columns."""
    a_cat = torch.cat([lora.lora_A.detach().to(dtype) for lora in loras], dim=1)
    bs = torch.cat([(float(lora.scale) * lora.lora_B.detach().float()).t() for lora in loras], dim=1).to(dtype)
    pad = -a_cat.shape[1] % _RANK_STEP
    if pad:
        a_cat = torch.nn.functional.pad(a_cat, (0, pad))
        bs = torch.nn.functional.pad(bs, (0, pad))
    return a_cat.contiguous(), bs.contiguous()


_DOWN_KERNEL_MAX_K = 4096


def down_fragments(a_cat: torch.Tensor) -> torch.Tensor:
    """``a_cat [K, R]`` (``K % 32 == 0``, ``R % 16 == 0``) in the order the
    down-projection kernel's matrix instruction consumes it:
    ``[R/16, K/32, 4, 16, 8]`` with ``af[f, s, q, c, e] = a_cat[32 s + 8 q + e, 16 f + c]``."""
    K, R = a_cat.shape
    if K % 32 or R % 16:
        raise ValueError(f"[down_fragments] a_cat must be [K, R] with K % 32 == 0 and R % 16 == 0, got {tuple(a_cat.shape)}")
    return a_cat.reshape(K // 32, 4, 8, R // 16, 16).permute(3, 0, 1, 4, 2).contiguous()


def _packed_for(owner: torch.nn.Module, loras: list[LoRALinear], dtype: torch.dtype):
    # rebuilt when an adapter's tensors are replaced or written in place, or a scale changes
    key = (dtype,) + tuple((id(lora), lora.lora_A.data_ptr(), lora.lora_A._version, lora.lora_B.data_ptr(),
                            lora.lora_B._version, float(lora.scale)) for lora in loras)
    cache = owner.__dict__.get("_packed_adapters")
    if cache is None or cache[0] != key:
        a_cat, bs = pack_adapters(loras, dtype)
        cache = (key, (a_cat, down_fragments(a_cat) if a_cat.shape[0] <= _DOWN_KERNEL_MAX_K else None, bs))
        owner.__dict__["_packed_adapters"] = cache
    return cache[1]


def _forward(owner: torch.nn.Module, base: torch.nn.Module, loras: list[LoRALinear], x: torch.Tensor) -> torch.Tensor:
    if not loras:
        return base(x)
    needs_grad = torch.is_grad_enabled() and (
        x.requires_grad or any(lora.lora_A.requires_grad or lora.lora_B.requires_grad for lora in loras))
    rank = sum(lora.lora_A.shape[1] for lora in loras)
    fused = (isinstance(base, QuantizedLinear) and x.is_cuda and not needs_grad and rank <= 1024
             and base.scales.dtype in (torch.bfloat16, torch.float16) and x.numel() > 0)
    if not fused:
        return _composed(base, loras, x)
    compute = base.scales.dtype
    a_cat, af, bs = _packed_for(owner, loras, compute)
    # t = x @ [lora_A_1 | lora_A_2 | ...], float32 sums rounded once.  Rows of up to 4096 elements (the hidden
    # sizes of the transformer blocks): one read of x in csrc/lora.hip, on a par with or ahead of the BLAS
    # library.  Longer rows (the MLP down-projections, K = 10240 .. 15360): the library's skinny split-K GEMM,
    # which is 1.2-1.6x faster there (the kernel streams such rows from memory at 3.5 TB/s only).
    K = x.shape[-1]
    if K <= _DOWN_KERNEL_MAX_K:
        t = _lib.ops().low_rank_down(x.to(compute).reshape(-1, K).contiguous(), af).reshape(*x.shape[:-1], bs.shape[1])
    else:
        t = torch.matmul(x.to(compute), a_cat)
    return core.quantized_matmul(x, base.weight, base.scales, base.biases, transpose=True, group_size=base.group_size,
                                 bits=base.bits, mode=base.mode, bias=base.bias, low_rank=(t, bs))


# ---- baking adapters into the base weights (for saving) -------------------------
def _delta(lora: LoRALinear) -> torch.Tensor:
    """``scale * (lora_A @ lora_B).T``, ``[out, in]``, in float32."""
    return float(lora.scale) * torch.matmul(lora.lora_A.detach().float(), lora.lora_B.detach().float()).t()


def _bake(base: torch.nn.Module, loras: list[LoRALinear], requantize: bool) -> None:
    if not hasattr(base, "weight") or not loras:
        return
    quantized = isinstance(base, QuantizedLinear)
    shape = (base.output_dims, base.input_dims) if quantized and requantize else tuple(base.weight.shape)
    deltas = []
    for lora in loras:
        delta = _delta(lora)
        if tuple(delta.shape) != shape:
            print(f"⚠️  Skipping LoRA bake due to shape mismatch: weight {shape} vs delta {tuple(delta.shape)}")
            continue
        deltas.append(delta)
    if not deltas:
        return
    if quantized:
        # all adapters at once, so that the weight is requantized a single time
        full = core.dequantize(base.weight, base.scales, base.biases, base.group_size, base.bits)
        baked = (full.float() + sum(deltas).to(full.device)).to(full.dtype)
        # written into the layer's own tensors: they may be views of a stack (nn.concat_quantized)
        for old, new in zip((base.weight, base.scales, base.biases),
                            core.quantize(baked, base.group_size, base.bits, base.mode)):
            old.copy_(new)
        return
    with torch.no_grad():
        for delta in deltas:   # one rounded add per adapter, as the reference does
            base.weight.add_(delta.to(device=base.weight.device, dtype=base.weight.dtype))


def bake_and_strip_lora(module: torch.nn.Module, requantize: bool = False) -> torch.nn.Module:
    """Replaces every ``LoRALinear`` / ``FusedLoRALinear`` below ``module`` by its
    base layer with the adapters added into the weight, as
    ``LoRASaver.bake_and_strip_lora``
    (src/mflux/models/common/lora/mapping/lora_saver.py:9-82) does before a
    model is saved: ``weight += (scale * lora_A @ lora_B).T`` in the weight's
    dtype.  Around a quantized base the reference's shapes do not match and it
    strips the wrapper without baking (``:75-77``), and so does this function
    by default; ``requantize=True`` instead dequantizes the base, adds the
    adapters in float32, rounds to the 16-bit type and quantizes again with the
    layer's group size and bits (lossy by one requantization).  Returns
    ``module`` (the base layer when ``module`` itself is a wrapper)."""
    def strip(obj: torch.nn.Module) -> torch.nn.Module:
        if isinstance(obj, FusedLoRALinear):
            _bake(obj.base_linear, [lora for lora in obj.loras if isinstance(lora, LoRALinear)], requantize)
            return obj.base_linear
        if isinstance(obj, LoRALinear):
            _bake(obj.linear, [obj], requantize)
            return obj.linear
        return obj

    module = strip(module)
    for name, child in list(module.named_children()):
        module._modules[name] = bake_and_strip_lora(child, requantize)
    return module
