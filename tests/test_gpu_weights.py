"""GPU: the quantize-on-the-fly and save -> reload flows end to end (the
counterpart of the reference's tests/model_saving/test_model_saving.py, which
checks that a reloaded 4-bit model reproduces the original's output
exactly)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


class Block(torch.nn.Module):
    def __init__(self, dim, hidden):
        super().__init__()
        from mflux_amd import nn as qnn

        self.to_q = qnn.Linear(dim, dim)
        self.mlp = torch.nn.ModuleList([qnn.Linear(dim, hidden), qnn.Linear(hidden, dim, bias=False)])
        self.norm = torch.nn.LayerNorm(dim)

    def forward(self, x):
        h = self.to_q(self.norm(x))
        return x + self.mlp[1](torch.nn.functional.gelu(self.mlp[0](h)))


class Tower(torch.nn.Module):
    def __init__(self, dim=256, hidden=512, n=2):
        super().__init__()
        from mflux_amd import nn as qnn

        self.inp = qnn.Linear(48, dim)  # 48 % 64 != 0: must stay float
        self.blocks = torch.nn.ModuleList([Block(dim, hidden) for _ in range(n)])

    def forward(self, x):
        x = self.inp(x)
        for b in self.blocks:
            x = b(x)
        return x


class Definition:
    @staticmethod
    def get_components():
        from mflux_amd import weights as W

        return [W.ComponentDefinition(name="transformer", hf_subdir="transformer")]

    @staticmethod
    def quantization_predicate(path, module):
        from mflux_amd import weights as W

        return W.group_aligned_predicate(path, module)


class Holder:
    def __init__(self, transformer):
        self.transformer = transformer


@pytest.mark.parametrize("bits", [3, 4, 5, 6, 8])
def test_quantize_on_the_fly_then_save_and_reload(tmp_path, oracle, bits):
    import numpy as np

    from gpu_util import raw
    from mflux_amd import nn as qnn
    from mflux_amd import weights as W

    torch.manual_seed(11 + bits)
    src = Tower().to(device="cuda", dtype=torch.bfloat16)
    float_weights = W.LoadedWeights(
        {"transformer": W.tree_unflatten([(k, v.clone()) for k, v in src.state_dict().items()])}, W.MetaData())

    # stored None + requested bits: weights are set first, then quantized on the device
    model = Tower().to(device="cuda", dtype=torch.bfloat16)
    got = W.WeightApplier.apply_and_quantize(float_weights, {"transformer": model}, bits, Definition)
    assert got == bits
    assert isinstance(model.inp, qnn.Linear)
    q = model.blocks[1].mlp[0]
    assert isinstance(q, qnn.QuantizedLinear) and q.bits == bits
    # the codes are those of the source weights, bit for bit
    exp = oracle.c_quantize(raw(src.blocks[1].mlp[0].weight), oracle.BF16, 64, bits)
    for e, g in zip(exp, (q.weight, q.scales, q.biases)):
        assert np.array_equal(raw(g), e)
    assert torch.equal(q.bias, src.blocks[1].mlp[0].bias)

    x = torch.randn(3, 70, 48, device="cuda").to(torch.bfloat16)
    y1 = model(x)
    W.save_model(Holder(model), bits, tmp_path, Definition)

    # reload without a request, and with a conflicting one
    for requested in (None, 8 if bits == 4 else 4):
        loaded = W.load_saved(Definition, tmp_path)
        fresh = Tower().to(device="cuda", dtype=torch.bfloat16)
        assert W.WeightApplier.apply_and_quantize(loaded, {"transformer": fresh}, requested, Definition) == bits
        for (ka, va), (kb, vb) in zip(model.state_dict().items(), fresh.state_dict().items()):
            assert ka == kb and vb.is_cuda and torch.equal(va.view(torch.uint8), vb.view(torch.uint8)), ka
        assert torch.equal(fresh(x), y1)


@pytest.mark.parametrize("M", [1, 512, 4096])
def test_concat_quantized_equals_the_separate_layers(M):
    """q, k, v stacked along N give the three outputs side by side.  Each output
    column depends on its own weight row only; the stacked shape may take a
    different kernel or K cut, so sums can differ in their last float32 bits:
    one bfloat16 ulp at the size of the row's largest output is allowed (the
    bias is added after the product is rounded, so a small output can carry the
    ulp of a larger product)."""
    import mflux_amd
    from mflux_amd import nn as qnn

    torch.manual_seed(11)
    K = 1024
    layers = [qnn.QuantizedLinear.from_linear(torch.nn.Linear(K, n, bias=(n != 768), device="cuda", dtype=torch.bfloat16),
                                              64, 4) for n in (1024, 768, 1024)]
    fused = qnn.concat_quantized(layers)
    x = torch.randn(M, K, device="cuda").to(torch.bfloat16)
    y = fused(x)
    parts = y.split([1024, 768, 1024], dim=-1)
    for part, layer in zip(parts, layers):
        ref = layer(x)
        assert part.shape == ref.shape
        bound = 2.0 ** -7 * ref.float().abs().amax(dim=-1, keepdim=True)
        assert torch.all((part.float() - ref.float()).abs() <= bound)
        assert (part != ref).float().mean() < 0.01   # and nearly all outputs are identical
