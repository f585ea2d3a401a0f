"""Host logic that needs no device: argument checking of the functional API,
the module tree walk of nn.quantize, the bit-width policy, and the saved
directory layout."""
import json

import pytest
import torch

import mflux_amd
from mflux_amd import nn as qnn
from mflux_amd import weights as W


# ---------------------------------------------------------------------------
# functional API: errors raised before any kernel is reached
# ---------------------------------------------------------------------------
def test_quantize_argument_errors():
    w = torch.zeros(4, 128, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="group size 48 is not supported"):
        mflux_amd.quantize(w, 48, 4)
    with pytest.raises(ValueError, match="number of bits 7 is not supported"):
        mflux_amd.quantize(w, 64, 7)
    with pytest.raises(ValueError, match="not implemented in this build"):
        mflux_amd.quantize(w, 64, 2)
    with pytest.raises(ValueError, match="at least 2 dimension"):
        mflux_amd.quantize(torch.zeros(128, dtype=torch.bfloat16), 64, 4)
    with pytest.raises(ValueError, match="divisible by the quantization group size"):
        mflux_amd.quantize(torch.zeros(4, 96, dtype=torch.bfloat16), 64, 4)
    with pytest.raises(ValueError, match="floating point"):
        mflux_amd.quantize(torch.zeros(4, 128, dtype=torch.int32), 64, 4)
    with pytest.raises(ValueError, match="mode"):
        mflux_amd.quantize(w, 64, 4, mode="mxfp4")


def test_no_cpu_fallback():
    """A CPU tensor is refused: the kernels are the only implementation."""
    w = torch.zeros(4, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        mflux_amd.quantize(w, 64, 4)
    wq = torch.zeros(8, 16, dtype=torch.uint32)
    s = torch.zeros(8, 2, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        mflux_amd.quantized_matmul(torch.zeros(2, 128, dtype=torch.bfloat16), wq, s, s)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        mflux_amd.dequantize(wq, s, s)


def test_quantized_matmul_shape_errors():
    wq = torch.zeros(8, 16, dtype=torch.uint32)
    s = torch.zeros(8, 2, dtype=torch.bfloat16)
    x = torch.zeros(2, 128, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="should be uint32"):
        mflux_amd.quantized_matmul(x, wq.to(torch.int32), s, s)
    with pytest.raises(ValueError, match="same shape"):
        mflux_amd.quantized_matmul(x, wq, s, s[:, :1])
    with pytest.raises(ValueError, match="incompatible"):
        mflux_amd.quantized_matmul(x, wq, s, s, bits=8)
    with pytest.raises(ValueError, match="does not match"):
        mflux_amd.quantized_matmul(x[:, :64], wq, s, s)


# ---------------------------------------------------------------------------
# nn.quantize: the tree walk and the predicate protocol
# ---------------------------------------------------------------------------
class Attn(torch.nn.Module):
    def __init__(self, dim):
        super().__init__()
        self.to_q = qnn.Linear(dim, dim)
        self.to_out = torch.nn.ModuleList([qnn.Linear(dim, dim), torch.nn.Identity()])
        self.norm = torch.nn.LayerNorm(dim)


class Net(torch.nn.Module):
    def __init__(self, dim=128):
        super().__init__()
        self.x_embedder = qnn.Linear(96, dim)  # 96 is not a multiple of 64
        self.blocks = torch.nn.ModuleList([Attn(dim), Attn(dim)])
        self.proj_out = qnn.Linear(dim, 64, bias=False)


def test_tree_walk_paths_and_predicate_arguments():
    net = Net()
    seen = []

    def predicate(path, module):
        seen.append((path, type(module).__name__))
        return False

    assert qnn.quantize(net, class_predicate=predicate) is net
    assert [p for p, _ in seen] == [
        "x_embedder", "blocks.0.to_q", "blocks.0.to_out.0", "blocks.0.to_out.1", "blocks.0.norm",
        "blocks.1.to_q", "blocks.1.to_out.0", "blocks.1.to_out.1", "blocks.1.norm", "proj_out",
    ]
    assert not any(isinstance(m, qnn.QuantizedLinear) for m in net.modules())


def test_quantize_replaces_selected_leaves_with_defaults_and_dict_answers():
    net = Net()
    calls = {}

    def fake_to_quantized(self, **kw):
        calls[id(self)] = kw
        with qnn.placeholder_quantization():
            return qnn.QuantizedLinear.from_linear(self, **kw)

    import unittest.mock as mock

    def predicate(path, module):
        if not hasattr(module, "to_quantized"):
            return False
        if path == "x_embedder":
            return False
        if path == "proj_out":
            return {"group_size": 32, "bits": 8}
        return True

    with mock.patch.object(qnn.Linear, "to_quantized", fake_to_quantized):
        qnn.quantize(net, bits=None, class_predicate=predicate)
    assert isinstance(net.x_embedder, qnn.Linear)
    q = net.blocks[1].to_out[0]
    assert isinstance(q, qnn.QuantizedLinear)
    assert (q.group_size, q.bits, q.mode) == (64, 4, "affine")           # None -> 64 / 4
    assert q.weight.dtype == torch.uint32 and tuple(q.weight.shape) == (128, 128 * 4 // 32)
    assert tuple(q.scales.shape) == tuple(q.biases.shape) == (128, 2)
    assert q.bias is not None and tuple(q.bias.shape) == (128,)
    assert (net.proj_out.group_size, net.proj_out.bits) == (32, 8)        # dict answer wins
    assert net.proj_out.bias is None
    assert tuple(net.proj_out.weight.shape) == (64, 128 * 8 // 32)
    assert set(k for kw in calls.values() for k in kw) <= {"group_size", "bits", "mode"}
    # what a LoRA wrapper reads back from a quantized layer
    assert q.weight.shape[1] * 32 // q.bits == 128 and q.input_dims == 128 and q.output_dims == 128
    assert not any(p.requires_grad for p in q.parameters())
    assert sorted(q.state_dict()) == ["bias", "biases", "scales", "weight"]


def test_predicate_true_on_unquantizable_module_raises():
    net = torch.nn.Sequential(torch.nn.LayerNorm(64))
    with pytest.raises(ValueError, match="Unable to quantize"):
        qnn.quantize(net, class_predicate=lambda p, m: True)
    with pytest.raises(ValueError, match="bool or a dict"):
        qnn.quantize(Net(), class_predicate=lambda p, m: "yes" if hasattr(m, "to_quantized") else False)


def test_default_predicate_hits_group_misaligned_layer():
    """With the default predicate the 96-wide layer is selected and refused by
    quantize, which is why model definitions carry shape-aware predicates."""
    with qnn.placeholder_quantization():
        with pytest.raises(ValueError, match="divisible by the quantization group size"):
            qnn.quantize(Net())
        net = Net()
        qnn.quantize(net, class_predicate=W.group_aligned_predicate, bits=8)
    assert isinstance(net.x_embedder, qnn.Linear)
    assert isinstance(net.proj_out, qnn.QuantizedLinear) and net.proj_out.bits == 8


def test_embedding_is_quantizable_and_walked():
    model = torch.nn.ModuleDict({"shared": qnn.Embedding(100, 128), "proj": qnn.Linear(128, 64)})
    with qnn.placeholder_quantization():
        qnn.quantize(model, bits=8)
    e = model["shared"]
    assert isinstance(e, qnn.QuantizedEmbedding) and isinstance(model["proj"], qnn.QuantizedLinear)
    assert (e.num_embeddings, e.dims, e.bits, e.group_size) == (100, 128, 8, 64)
    assert tuple(e.weight.shape) == (100, 32) and tuple(e.scales.shape) == (100, 2)
    assert sorted(e.state_dict()) == ["biases", "scales", "weight"]
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        e(torch.tensor([1, 2]))
    with pytest.raises(ValueError, match="divisible"):
        qnn.QuantizedEmbedding(10, 96)
    plain = qnn.Embedding(10, 64)
    assert torch.equal(plain.as_linear(torch.ones(1, 64)), torch.ones(1, 64) @ plain.weight.T)


def test_concat_quantized_stacks_rows_and_checks_compatibility():
    a = qnn.QuantizedLinear(128, 64, bias=True, bits=4)
    b = qnn.QuantizedLinear(128, 32, bias=False, bits=4)
    c = qnn.QuantizedLinear(128, 16, bias=True, bits=4)
    a.weight.fill_(1), b.weight.fill_(2), c.weight.fill_(3)
    a.bias.fill_(0.5), c.bias.fill_(-1.0)
    fused = qnn.concat_quantized([a, b, c])
    assert isinstance(fused, qnn.QuantizedLinear) and (fused.input_dims, fused.output_dims) == (128, 112)
    assert (fused.group_size, fused.bits, fused.mode) == (64, 4, "affine")
    assert fused.weight.dtype == torch.uint32 and tuple(fused.weight.shape) == (112, 16)
    assert tuple(fused.scales.shape) == (112, 2) and tuple(fused.biases.shape) == (112, 2)
    assert fused.weight.view(torch.int32)[:, 0].tolist() == [1] * 64 + [2] * 32 + [3] * 16
    assert fused.bias.tolist() == [0.5] * 64 + [0.0] * 32 + [-1.0] * 16     # a missing bias is zeros
    assert sorted(fused.state_dict()) == ["bias", "biases", "scales", "weight"]
    assert qnn.concat_quantized([b, b]).bias is None
    with pytest.raises(ValueError, match="must share"):
        qnn.concat_quantized([a, qnn.QuantizedLinear(128, 64, bits=8)])
    with pytest.raises(ValueError, match="must share"):
        qnn.concat_quantized([a, qnn.QuantizedLinear(256, 64, bits=4)])
    with pytest.raises(ValueError, match="expected QuantizedLinear"):
        qnn.concat_quantized([a, torch.nn.Linear(128, 64)])
    with pytest.raises(ValueError, match="at least one"):
        qnn.concat_quantized([])


def test_concat_quantized_share_storage_turns_the_layers_into_views():
    a = qnn.QuantizedLinear(128, 64, bias=True, bits=8)
    b = qnn.QuantizedLinear(128, 32, bias=False, bits=8)
    a.weight.fill_(7), b.weight.fill_(9)
    a.scales.fill_(0.5), b.scales.fill_(0.25)
    a.bias.fill_(1.5)
    fused = qnn.concat_quantized([a, b], share_storage=True)
    for layer, rows in ((a, slice(0, 64)), (b, slice(64, 96))):
        for name in ("weight", "scales", "biases"):
            view, whole = getattr(layer, name), getattr(fused, name)
            assert view.untyped_storage().data_ptr() == whole.untyped_storage().data_ptr()
            assert view.is_contiguous() and torch.equal(view.view(torch.uint8), whole[rows].view(torch.uint8))
    assert a.bias.untyped_storage().data_ptr() == fused.bias.untyped_storage().data_ptr() and b.bias is None
    assert a.weight.view(torch.int32)[0, 0] == 7 and b.weight.view(torch.int32)[0, 0] == 9
    assert a.bias.tolist() == [1.5] * 64 and fused.bias.tolist() == [1.5] * 64 + [0.0] * 32
    assert sorted(a.state_dict()) == ["bias", "biases", "scales", "weight"]     # still the four saved tensors
    fused.scales[:64].fill_(2.0)                                                # one memory
    assert a.scales[0, 0] == 2.0


def test_quantized_linear_constructor_on_cpu_is_a_placeholder():
    q = qnn.QuantizedLinear(256, 64, bias=True, group_size=None, bits=8)
    assert (q.group_size, q.bits) == (64, 8)
    assert tuple(q.weight.shape) == (64, 64) and q.weight.dtype == torch.uint32
    assert "input_dims=256, output_dims=64, bias=True, group_size=64, bits=8" in repr(q)
    with pytest.raises(ValueError, match="divisible"):
        qnn.QuantizedLinear(100, 64)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        q(torch.zeros(1, 256, dtype=torch.bfloat16))


# ---------------------------------------------------------------------------
# bit-width policy: every stored x requested combination the reference tests
# ---------------------------------------------------------------------------
LEVELS = [None, 3, 4, 5, 6, 8]


@pytest.mark.parametrize("stored", LEVELS)
@pytest.mark.parametrize("requested", LEVELS)
def test_resolution_table(stored, requested):
    bits, warning = W.QuantizationResolution.resolve(stored=stored, requested=requested)
    if stored is None:
        assert bits == requested and warning is None
    else:
        assert bits == stored
        if requested is None or requested == stored:
            assert warning is None
        else:
            assert f"{stored}-bit" in warning and f"-q {requested}" in warning


# ---------------------------------------------------------------------------
# trees, update, ordering, save / reload
# ---------------------------------------------------------------------------
def test_tree_flatten_unflatten_round_trip():
    t = {"a": {"b": [{"w": 1}, {"w": 2, "v": 3}]}, "c": 4}
    flat = W.tree_flatten(t)
    assert flat == [("a.b.0.w", 1), ("a.b.1.w", 2), ("a.b.1.v", 3), ("c", 4)]
    assert W.tree_unflatten(flat) == t


class Definition:
    @staticmethod
    def get_components():
        return [W.ComponentDefinition(name="transformer", hf_subdir="transformer"),
                W.ComponentDefinition(name="vae", hf_subdir="vae", skip_quantization=True)]

    quantization_predicate = staticmethod(W.group_aligned_predicate)


class Pipeline:
    def __init__(self):
        self.transformer = Net()
        self.vae = torch.nn.Sequential(qnn.Linear(64, 64))


def _fill_fake_codes(model, seed=0):
    g = torch.Generator().manual_seed(seed)
    for m in model.modules():
        if isinstance(m, qnn.QuantizedLinear):
            m.weight = torch.randint(0, 2 ** 31 - 1, m.weight.shape, generator=g, dtype=torch.int32).view(torch.uint32)
            m.scales = torch.randn(m.scales.shape, generator=g).to(m.scales.dtype)
            m.biases = torch.randn(m.biases.shape, generator=g).to(m.biases.dtype)


def test_save_reload_round_trip_and_layout(tmp_path):
    pipe = Pipeline()
    pipe.transformer.to(torch.bfloat16)
    with qnn.placeholder_quantization():
        qnn.quantize(pipe.transformer, class_predicate=Definition.quantization_predicate, bits=4)
    _fill_fake_codes(pipe.transformer)
    W.save_model(pipe, 4, tmp_path, Definition)

    index = json.load(open(tmp_path / "transformer" / "model.safetensors.index.json"))
    assert index["metadata"] == {"quantization_level": "4", "mflux_version": mflux_amd.__version__}
    assert set(index["weight_map"].values()) == {"0.safetensors"}
    assert "blocks.0.to_out.0.scales" in index["weight_map"] and "x_embedder.weight" in index["weight_map"]
    from safetensors import safe_open

    with safe_open(str(tmp_path / "transformer" / "0.safetensors"), framework="pt") as f:
        assert f.metadata()["quantization_level"] == "4"
        assert f.get_slice("blocks.0.to_q.weight").get_dtype() == "U32"
        assert f.get_slice("blocks.0.to_q.scales").get_dtype() == "BF16"
        assert f.get_slice("x_embedder.weight").get_dtype() == "BF16"

    tree, level, version = W.try_load_saved_format(tmp_path / "vae")
    assert level == 4 and version == mflux_amd.__version__
    assert isinstance(tree, dict) and "0" in tree or isinstance(tree, list)

    # reload into a fresh pipeline: stored level wins over the request, with a warning
    loaded = W.load_saved(Definition, tmp_path)
    assert loaded.meta_data.quantization_level == 4
    fresh = Pipeline()
    fresh.transformer.to(torch.bfloat16)
    bits = W.WeightApplier.apply_and_quantize(loaded, {"transformer": fresh.transformer, "vae": fresh.vae}, 8,
                                              Definition)
    assert bits == 4
    a, b = pipe.transformer.state_dict(), fresh.transformer.state_dict()
    assert list(a) == list(b)
    for k in a:
        assert a[k].dtype == b[k].dtype and torch.equal(a[k].view(torch.uint8), b[k].view(torch.uint8)), k
    assert isinstance(fresh.vae[0], qnn.Linear)  # skip_quantization component stays float
    assert torch.equal(fresh.vae[0].weight, pipe.vae[0].weight)


def test_stored_quantized_component_with_missing_codes_is_refused(tmp_path):
    pipe = Pipeline()
    with qnn.placeholder_quantization():
        qnn.quantize(pipe.transformer, class_predicate=Definition.quantization_predicate, bits=8)
    sd = {k: v for k, v in pipe.transformer.state_dict().items() if not k.startswith("blocks.1.to_q.")}
    weights = W.LoadedWeights({"transformer": W.tree_unflatten(list(sd.items()))}, W.MetaData(8, "x"))
    comp = Definition.get_components()[0]
    with pytest.raises(ValueError, match="packed tensors are missing"):
        W.WeightApplier.apply_and_quantize_single(weights, Net(), comp, None, Definition.quantization_predicate)
    with pytest.raises(ValueError, match="No weights found"):
        W.WeightApplier.apply_and_quantize_single(W.LoadedWeights({}, W.MetaData()), Net(), comp, None)


def test_unquantized_apply_keeps_float_layers():
    src = Net()
    weights = W.LoadedWeights({"transformer": W.tree_unflatten(list(src.state_dict().items()))}, W.MetaData())
    dst = Net()
    bits = W.WeightApplier.apply_and_quantize(weights, {"transformer": dst}, None, Definition)
    assert bits is None
    for (ka, va), (kb, vb) in zip(src.state_dict().items(), dst.state_dict().items()):
        assert ka == kb and torch.equal(va, vb)
    assert dst.proj_out.weight.requires_grad


def test_split_weights_greedy_order():
    t = {f"t{i}": torch.zeros(n, dtype=torch.uint8) for i, n in enumerate([60, 50, 30, 200, 10, 10])}
    shards = W.split_weights(t, max_bytes=100)
    assert [list(s) for s in shards] == [["t0"], ["t1", "t2"], ["t3"], ["t4", "t5"]]
    assert W.split_weights({}, 100) == []
    # a first tensor beyond the limit: the reference closes the still empty shard in front of it
    # (model_saver.py:92-95 has no "if shard"), so its own shard is number 1; a last one is never empty
    big = {"a": torch.zeros(150, dtype=torch.uint8), "b": torch.zeros(10, dtype=torch.uint8)}
    assert [list(s) for s in W.split_weights(big, max_bytes=100)] == [[], ["a"], ["b"]]
    assert [list(s) for s in W.split_weights({"a": torch.zeros(150, dtype=torch.uint8)}, max_bytes=100)] == [[], ["a"]]


def test_foreign_directory_is_not_our_format(tmp_path):
    from safetensors.torch import save_file

    assert W.try_load_saved_format(tmp_path / "nope") == (None, None, None)
    (tmp_path / "empty").mkdir()
    assert W.try_load_saved_format(tmp_path / "empty") == (None, None, None)
    (tmp_path / "hf").mkdir()
    save_file({"w": torch.zeros(2)}, str(tmp_path / "hf" / "model.safetensors"))
    assert W.try_load_saved_format(tmp_path / "hf") == (None, None, None)
    save_file({"w": torch.zeros(2)}, str(tmp_path / "hf" / "model.safetensors"),
              metadata={"quantization_level": "None", "mflux_version": "0.1"})
    tree, level, version = W.try_load_saved_format(tmp_path / "hf")
    assert level is None and version == "0.1" and torch.equal(tree["w"], torch.zeros(2))


def test_bake_and_strip_lora_on_float_and_quantized_bases(capsys):
    """Wrappers are replaced by their bases wherever they sit in the tree; a
    float base gets weight += (scale * A @ B).T; a quantized base is stripped
    without baking, with the reference's warning (lora_saver.py:75-77)."""
    from mflux_amd.lora import FusedLoRALinear, LoRALinear, bake_and_strip_lora

    torch.manual_seed(0)

    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.proj = LoRALinear.from_linear(torch.nn.Linear(32, 16, dtype=torch.float32), r=4, scale=0.5)
            lin = torch.nn.Linear(32, 8, dtype=torch.float32)
            self.heads = torch.nn.ModuleList([
                FusedLoRALinear(lin, [LoRALinear.from_linear(lin, r=2, scale=1.0), LoRALinear.from_linear(lin, r=3, scale=-2.0)]),
                torch.nn.Linear(8, 8),
            ])
            self.q = LoRALinear.from_linear(qnn.QuantizedLinear(64, 16, bias=False, bits=4), r=4)

    net = Block()
    x = torch.randn(5, 32)
    want_proj, want_head = net.proj(x), net.heads[0](x)
    w_before = net.heads[0].base_linear.weight.detach().clone()
    loras = list(net.heads[0].loras)
    packed_before = net.q.linear.weight.clone()
    out = bake_and_strip_lora(net)
    assert out is net
    assert type(net.proj) is torch.nn.Linear and type(net.heads[0]) is torch.nn.Linear
    assert isinstance(net.q, qnn.QuantizedLinear) and torch.equal(net.q.weight, packed_before)
    assert "Skipping LoRA bake due to shape mismatch" in capsys.readouterr().out
    delta = sum(l.scale * (l.lora_A.float() @ l.lora_B.float()).t() for l in loras)
    assert torch.allclose(net.heads[0].weight, w_before + delta, atol=1e-6)
    assert torch.allclose(net.proj(x), want_proj, atol=1e-5) and torch.allclose(net.heads[0](x), want_head, atol=1e-5)
    # a wrapper passed in directly comes back as its baked base
    top = LoRALinear.from_linear(torch.nn.Linear(8, 4, dtype=torch.float32), r=2)
    assert type(bake_and_strip_lora(top)) is torch.nn.Linear


def test_save_model_bakes_and_strips_lora_wrappers(tmp_path):
    """A model still wrapped in LoRA layers is saved as its baked base model
    (model_saver.py:38-41 calls LoRASaver.bake_and_strip_lora first), so the
    saved keys are the base model's and a fresh model reloads them all."""
    from mflux_amd.lora import LoRALinear

    torch.manual_seed(3)
    pipe = Pipeline()
    x = torch.randn(3, pipe.transformer.x_embedder.in_features)
    pipe.transformer.x_embedder = LoRALinear.from_linear(pipe.transformer.x_embedder, r=4, scale=0.7)
    with torch.no_grad():
        pipe.transformer.x_embedder.lora_B.normal_()
    want = pipe.transformer.x_embedder(x)
    W.save_model(pipe, None, tmp_path, Definition)
    assert type(pipe.transformer.x_embedder) is qnn.Linear           # stripped in place, as the reference does
    index = json.load(open(tmp_path / "transformer" / "model.safetensors.index.json"))
    assert "x_embedder.weight" in index["weight_map"]
    assert not any("lora" in k or ".linear." in k for k in index["weight_map"])
    fresh = Pipeline()
    loaded = W.load_saved(Definition, tmp_path)
    W.WeightApplier.apply_and_quantize(loaded, {"transformer": fresh.transformer, "vae": fresh.vae}, None, Definition)
    assert torch.allclose(fresh.transformer.x_embedder(x), want, atol=1e-5)


def test_update_module_writes_into_shared_storage():
    """Layers stacked with concat_quantized(share_storage=True) are views of the
    stack: loading stored tensors of the same shape afterwards must reach the
    stack too (copied in place), not detach the layer from it."""
    with qnn.placeholder_quantization():
        a = qnn.QuantizedLinear(64, 8, bias=False, bits=4)
        b = qnn.QuantizedLinear(64, 16, bias=False, bits=4)
    model = torch.nn.ModuleDict({"a": a, "b": b})
    stack = qnn.concat_quantized([a, b], share_storage=True)
    new_w = torch.arange(16 * 8, dtype=torch.int32).reshape(16, 8).view(torch.uint32)
    new_s = torch.full((16, 1), 0.5, dtype=b.scales.dtype)
    done = W.update_module(model, {"b": {"weight": new_w, "scales": new_s}})
    assert done == {"b.weight", "b.scales"}
    assert torch.equal(stack.weight[8:].view(torch.int32), new_w.view(torch.int32))
    assert torch.equal(stack.scales[8:], new_s)
    assert b.weight.data_ptr() == stack.weight[8:].data_ptr()
    # a value of another shape still replaces the tensor (a float weight becoming packed codes)
    lin = torch.nn.ModuleDict({"l": qnn.Linear(64, 8, bias=False)})
    W.update_module(lin, {"l": {"weight": torch.zeros(8, 8, dtype=torch.int32).view(torch.uint32)}})
    assert lin["l"].weight.dtype == torch.uint32 and tuple(lin["l"].weight.shape) == (8, 8)


def test_down_projection_fragment_order():
    """The stacked lora_A as the down-projection kernel reads it: fragment f, step
    s, lane 16 q + c holds a_cat[32 s + 8 q .. + 7, 16 f + c]."""
    import numpy as np
    import torch

    from mflux_amd.lora import down_fragments

    a = torch.arange(96 * 48, dtype=torch.float32).reshape(96, 48)
    af = down_fragments(a)
    assert tuple(af.shape) == (3, 3, 4, 16, 8) and af.is_contiguous()
    f, s, q, c, e = np.indices(af.shape)
    assert np.array_equal(af.numpy(), a.numpy()[32 * s + 8 * q + e, 16 * f + c])
    with pytest.raises(ValueError):
        down_fragments(torch.zeros(40, 16))
    with pytest.raises(ValueError):
        down_fragments(torch.zeros(64, 8))
