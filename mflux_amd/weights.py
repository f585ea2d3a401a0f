"""Host side of the quantized-weight life cycle: which bit width wins, in what
order weights are set and layers quantized, and the directory layout a
quantized model is saved to and reloaded from.

Mirrors, on torch modules, the callers either side of the kernels:
  - ``QuantizationResolution.resolve``
    (src/mflux/models/common/resolution/quantization_resolution.py:18-52),
  - ``WeightApplier.apply_and_quantize[_single]``
    (src/mflux/models/common/weights/loading/weight_applier.py:15-103),
  - ``ModelSaver._save_weights`` / ``_split_weights``
    (src/mflux/models/common/weights/saving/model_saver.py:50-99),
  - ``WeightLoader._try_load_mflux_format``
    (src/mflux/models/common/weights/loading/weight_loader.py:145-179).

Saved layout, per component: ``<base>/<subdir>/{0,1,...}.safetensors`` with
string metadata ``quantization_level`` and ``mflux_version``, tensors named by
their dotted parameter path (``blocks.0.attn.to_q.weight`` uint32,
``....scales`` / ``....biases`` / ``....bias`` in the 16-bit float type), shards
of at most 2 GiB filled greedily in parameter order, and a
``model.safetensors.index.json`` mapping every tensor to its shard.
"""
from __future__ import annotations

import json
import logging
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any, Callable, Iterable

import torch

from . import nn as qnn

logger = logging.getLogger(__name__)

FORMAT_VERSION_KEY = "mflux_version"
QUANTIZATION_KEY = "quantization_level"
MAX_SHARD_BYTES = 2 << 30


# ---------------------------------------------------------------------------
# which bit width applies
# ---------------------------------------------------------------------------
class QuantizationResolution:
    """``resolve(stored, requested) -> (bits, warning)``.

    Nothing stored and nothing requested: no quantization.  Nothing stored:
    quantize on the fly at the requested width.  Weights stored quantized: the
    stored width always wins; a different requested width is ignored with a
    warning."""

    @staticmethod
    def resolve(stored: int | None, requested: int | None) -> tuple[int | None, str | None]:
        if stored is None:
            return requested, None
        warning = None
        if requested is not None and requested != stored:
            warning = f"Model is pre-quantized at {stored}-bit. Ignoring -q {requested} flag."
        logger.debug("quantization resolution: stored=%s requested=%s -> %s", stored, requested, stored)
        return stored, warning


# ---------------------------------------------------------------------------
# nested weight trees <-> dotted names
# ---------------------------------------------------------------------------
def tree_flatten(tree: Any, prefix: str = "") -> list[tuple[str, Any]]:
    """Nested dicts / lists of tensors -> [(dotted path, tensor)], list indices
    spelled as numbers (``blocks.0.attn``)."""
    out: list[tuple[str, Any]] = []
    if isinstance(tree, dict):
        for k, v in tree.items():
            out.extend(tree_flatten(v, f"{prefix}.{k}" if prefix else str(k)))
    elif isinstance(tree, (list, tuple)):
        for i, v in enumerate(tree):
            out.extend(tree_flatten(v, f"{prefix}.{i}" if prefix else str(i)))
    else:
        out.append((prefix, tree))
    return out


def tree_unflatten(items: Iterable[tuple[str, Any]]) -> Any:
    """Inverse of ``tree_flatten``: path components that are all numbers at one
    level become a list (holes filled with empty dicts)."""
    items = list(items)
    if len(items) == 1 and items[0][0] == "":
        return items[0][1]
    children: dict[str, list[tuple[str, Any]]] = {}
    for path, value in items:
        head, _, rest = path.partition(".")
        children.setdefault(head, []).append((rest, value))
    built = {k: tree_unflatten(v) for k, v in children.items()}
    if built and all(k.isdigit() for k in built):
        size = max(int(k) for k in built) + 1
        as_list: list[Any] = [{} for _ in range(size)]
        for k, v in built.items():
            as_list[int(k)] = v
        return as_list
    return built


def update_module(model: torch.nn.Module, tree: Any, strict: bool = False) -> set[str]:
    """Sets parameters and buffers of ``model`` from a nested tree (or a flat
    ``{dotted path: tensor}`` dict).  A value of the stored tensor's shape and
    dtype is copied into it, so that views of that storage stay valid (the
    layers of ``nn.concat_quantized(..., share_storage=True)`` are views of the
    stack); any other value replaces the stored tensor, so dtype and shape
    follow it (a quantized layer's ``weight`` is uint32 of a different shape
    than the float one).  Paths that name nothing in the model are skipped
    unless ``strict``.  Returns the set of paths that were set."""
    done: set[str] = set()
    for path, value in tree_flatten(tree):
        if not isinstance(value, torch.Tensor):
            raise ValueError(f"weight '{path}' is a {type(value).__name__}, not a tensor")
        owner_path, _, name = path.rpartition(".")
        try:
            owner = model.get_submodule(owner_path) if owner_path else model
        except AttributeError:
            owner = None
        if owner is None or not (name in owner._parameters or name in owner._buffers):
            if strict:
                raise ValueError(f"weight '{path}' does not match any parameter of the model")
            continue
        params = name in owner._parameters
        old = owner._parameters[name] if params else owner._buffers[name]
        if old is not None and old.shape == value.shape and old.dtype == value.dtype:
            with torch.no_grad():
                old.copy_(value)
        elif params:
            if old is not None:
                value = value.to(old.device)
            trainable = bool(old is not None and old.requires_grad and value.is_floating_point())
            owner._parameters[name] = torch.nn.Parameter(value, requires_grad=trainable)
        else:
            owner._buffers[name] = value.to(old.device) if old is not None else value
        done.add(path)
    return done


# ---------------------------------------------------------------------------
# set weights and quantize, in the order that keeps stored codes intact
# ---------------------------------------------------------------------------
@dataclass
class MetaData:
    quantization_level: int | None = None
    mflux_version: str | None = None


@dataclass
class LoadedWeights:
    components: dict[str, Any]
    meta_data: MetaData = field(default_factory=MetaData)


@dataclass
class ComponentDefinition:
    """The fields of the reference's component description that this path
    reads (src/mflux/models/common/weights/loading/weight_definition.py:32-48)."""
    name: str
    hf_subdir: str
    model_attr: str | None = None
    skip_quantization: bool = False
    weight_subkey: str | None = None


def default_predicate(path: str, module: torch.nn.Module) -> bool:
    return hasattr(module, "to_quantized")


def group_aligned_predicate(path: str, module: torch.nn.Module, group_size: int = 64) -> bool:
    """Skips layers whose input width is not a multiple of the group size
    (src/mflux/models/krea2/weights/krea2_weight_definition.py:84-90)."""
    if not hasattr(module, "to_quantized"):
        return False
    weight = getattr(module, "weight", None)
    return weight is not None and weight.shape[-1] % group_size == 0


def _quantized_paths(model: torch.nn.Module) -> list[str]:
    return [p for p, m in model.named_modules() if isinstance(m, (qnn.QuantizedLinear, qnn.QuantizedEmbedding))]


def _quantize_for_stored(model: torch.nn.Module, predicate: Callable, bits: int) -> list[str]:
    """Turns the selected layers into quantized layers of the right shapes
    WITHOUT running the quantize kernel: the stored codes are about to replace
    whatever the layers hold.  Returns the paths that now expect stored
    tensors."""
    before = set(_quantized_paths(model))
    with qnn.placeholder_quantization():
        qnn.quantize(model, class_predicate=predicate, bits=bits)
    return [p for p in _quantized_paths(model) if p not in before]


def _check_filled(component: str, expected: list[str], done: set[str]) -> None:
    missing = [f"{p}.{t}" for p in expected for t in ("weight", "scales", "biases") if f"{p}.{t}" not in done]
    if missing:
        raise ValueError(
            f"component '{component}' is stored quantized but {len(missing)} packed tensors are missing, "
            f"first: {missing[:3]}"
        )


class WeightApplier:
    @staticmethod
    def apply_and_quantize_single(weights: LoadedWeights, model: torch.nn.Module, component: ComponentDefinition,
                                  quantize_arg: int | None, quantization_predicate: Callable | None = None):
        stored = weights.meta_data.quantization_level
        tree = weights.components.get(component.name)
        if tree is None:
            raise ValueError(f"No weights found for component: {component.name}")
        predicate = quantization_predicate or default_predicate
        bits, warning = QuantizationResolution.resolve(stored=stored, requested=quantize_arg)
        if warning:
            print(f"⚠️  {warning}")
        WeightApplier._apply_one(component.name, model, tree, bits, stored, component.skip_quantization, predicate)
        return bits

    @staticmethod
    def apply_and_quantize(weights: LoadedWeights, models: dict[str, torch.nn.Module], quantize_arg: int | None,
                           weight_definition) -> int | None:
        stored = weights.meta_data.quantization_level
        components = {c.name: c for c in weight_definition.get_components()}
        bits, warning = QuantizationResolution.resolve(stored=stored, requested=quantize_arg)
        if warning:
            print(f"⚠️  {warning}")
        for name, model in models.items():
            component = components.get(name)
            tree = weights.components.get(name)
            if tree is not None and component is not None and component.weight_subkey is not None \
                    and isinstance(tree, dict):
                tree = tree.get(component.weight_subkey, tree)
            skip = bool(component and component.skip_quantization)
            WeightApplier._apply_one(name, model, tree, bits, stored, skip, weight_definition.quantization_predicate)
        return bits

    @staticmethod
    def _apply_one(name: str, model: torch.nn.Module, tree: Any, bits: int | None, stored: int | None, skip: bool,
                   predicate: Callable) -> None:
        if bits is None or skip:
            if tree is not None:
                update_module(model, tree, strict=False)
        elif stored is None:
            # float weights in, then quantize them on the device
            if tree is not None:
                update_module(model, tree, strict=False)
            qnn.quantize(model, class_predicate=predicate, bits=bits)
        else:
            # stored codes: give the layers their quantized shape first, then
            # drop the stored tensors in
            expected = _quantize_for_stored(model, predicate, bits)
            done = update_module(model, tree, strict=False) if tree is not None else set()
            _check_filled(name, expected, done)


# ---------------------------------------------------------------------------
# saving and reloading
# ---------------------------------------------------------------------------
def library_version() -> str:
    from . import __version__

    return __version__


def split_weights(weights: dict[str, torch.Tensor], max_bytes: int = MAX_SHARD_BYTES) -> list[dict]:
    """Greedy, order-preserving shards, statement for statement
    ``ModelSaver._split_weights``
    (src/mflux/models/common/weights/saving/model_saver.py:86-99): a tensor that
    would take the running shard past ``max_bytes`` closes it and starts the
    next one.  As in the reference the running shard is closed even when it is
    still empty, so a first tensor larger than ``max_bytes`` leaves an empty
    shard 0 in front of its own; only a trailing empty shard is dropped."""
    shards: list[dict] = []
    shard: dict = {}
    size = 0
    for key, value in weights.items():
        nbytes = value.numel() * value.element_size()
        if size + nbytes > max_bytes:
            shards.append(shard)
            shard, size = {}, 0
        shard[key] = value
        size += nbytes
    if shard:
        shards.append(shard)
    return shards


def save_weights(base_path: str | Path, bits: int | None, model: torch.nn.Module, subdir: str,
                 max_bytes: int = MAX_SHARD_BYTES) -> list[Path]:
    from safetensors.torch import save_file

    path = Path(base_path) / subdir
    path.mkdir(parents=True, exist_ok=True)
    weights = {k: v.detach().contiguous().cpu() for k, v in model.state_dict().items()}
    meta = {QUANTIZATION_KEY: str(bits), FORMAT_VERSION_KEY: library_version()}
    weight_map: dict[str, str] = {}
    written: list[Path] = []
    for i, shard in enumerate(split_weights(weights, max_bytes)):
        filename = f"{i}.safetensors"
        save_file(shard, str(path / filename), metadata=meta)
        written.append(path / filename)
        for key in shard:
            weight_map[key] = filename
    with open(path / "model.safetensors.index.json", "w") as f:
        json.dump({"metadata": meta, "weight_map": weight_map}, f, indent=2)
    return written


def save_model(model: Any, bits: int | None, base_path: str | Path, weight_definition) -> None:
    """One directory per component, named by the component's ``hf_subdir``; the
    component is the attribute ``model_attr`` (or ``name``) of ``model``.  As
    ``ModelSaver.save_model`` does
    (src/mflux/models/common/weights/saving/model_saver.py:38-41), LoRA wrappers
    are baked into their base layers and stripped first (in place: the model
    keeps the baked layers), so that the saved keys are the base model's."""
    from .lora import bake_and_strip_lora

    for c in weight_definition.get_components():
        attr = c.model_attr or c.name
        component = getattr(model, attr, None)
        if component is not None:
            stripped = bake_and_strip_lora(component)
            if stripped is not component:  # the component itself was a wrapper
                setattr(model, attr, stripped)
            save_weights(base_path, bits, stripped, c.hf_subdir)


def try_load_saved_format(path: str | Path, device: str | torch.device = "cpu"):
    """Reads a component directory written by ``save_weights``.  Returns
    ``(tree, quantization_level, version)``; ``(None, None, None)`` when the
    directory is missing, holds no safetensors file, or its first file carries
    neither metadata key (then it is someone else's format)."""
    from safetensors import safe_open

    path = Path(path)
    if not path.exists():
        return None, None, None
    shard_files = sorted(f for f in path.glob("*.safetensors") if not f.name.startswith("._"))
    if not shard_files:
        return None, None, None
    with safe_open(str(shard_files[0]), framework="pt", device="cpu") as f:
        meta = f.metadata() or {}
    level_str = meta.get(QUANTIZATION_KEY)
    version = meta.get(FORMAT_VERSION_KEY)
    if level_str is None and version is None:
        return None, None, None
    level = None if level_str in (None, "None", "null", "") else int(level_str)
    tensors: dict[str, torch.Tensor] = {}
    for shard in shard_files:
        with safe_open(str(shard), framework="pt", device=str(device)) as f:
            for key in f.keys():
                tensors[key] = f.get_tensor(key)
    return tree_unflatten(list(tensors.items())), level, version


def load_saved(weight_definition, base_path: str | Path, device: str | torch.device = "cpu") -> LoadedWeights:
    """All components of a saved model; the quantization level is the first
    one found."""
    components: dict[str, Any] = {}
    meta = MetaData()
    for c in weight_definition.get_components():
        tree, level, version = try_load_saved_format(Path(base_path) / c.hf_subdir, device)
        if tree is None:
            raise ValueError(f"component '{c.name}': nothing in the saved format under {Path(base_path) / c.hf_subdir}")
        components[c.name] = tree
        if meta.quantization_level is None and level is not None:
            meta = MetaData(quantization_level=level, mflux_version=version)
    return LoadedWeights(components=components, meta_data=meta)
