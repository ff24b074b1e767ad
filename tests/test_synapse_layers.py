"""The dense synapse layer (slayer.synapse.Dense; synapse/layer.py:72-175 in the reference) is the matrix product
the reference writes as a convolution whose kernel covers the whole input: against F.conv3d as the reference calls
it, for the three ways of naming the input (neurons, (width, height), (width, height, channels)), with a weight
pre-hook and weight normalisation, and the gradients through it."""
import torch
import torch.nn.functional as F

import lava_dl_amd.slayer as slayer


def _reference(layer, weight, x):
    if x.dim() == 3:
        n, t = x.shape[0], x.shape[-1]
        return F.conv3d(x.reshape(n, -1, 1, 1, t), weight, None, layer.stride, layer.padding, layer.dilation,
                        layer.groups).reshape(n, -1, t)
    return F.conv3d(x, weight, None, layer.stride, layer.padding, layer.dilation, layer.groups)


def test_dense_is_the_references_convolution():
    gen = torch.Generator().manual_seed(5)
    quant = lambda w: (w * 16).round() / 16
    cases = [(slayer.synapse.Dense(6, 4, weight_scale=2, pre_hook_fx=quant), (3, 6, 11), (4, 6, 1, 1, 1)),
             (slayer.synapse.Dense((3, 5), 7), (2, 1, 5, 3, 9), (7, 1, 5, 3, 1)),
             (slayer.synapse.Dense((3, 5, 2), 7), (2, 2, 5, 3, 9), (7, 2, 5, 3, 1)),
             (slayer.synapse.Dense((2, 2, 3), 5), (2, 3, 4, 6, 8), (5, 3, 2, 2, 1))]     # image larger than the kernel
    for layer, shape, wshape in cases:
        assert tuple(layer.shape) == wshape and layer.bias is None and layer.complex is False
        x = torch.randn(shape, generator=gen).requires_grad_()
        y = layer(x)
        weight = layer.weight if layer.pre_hook_fx is None else layer.pre_hook_fx(layer.weight)
        want = _reference(layer, weight, x)
        assert y.shape == want.shape
        assert torch.allclose(y, want, rtol=1e-5, atol=1e-6)
        g = torch.randn(y.shape, generator=gen)
        gx, gw = torch.autograd.grad(y, (x, layer.weight), g)
        rx, rw = torch.autograd.grad(want, (x, layer.weight), g)
        assert torch.allclose(gx, rx, rtol=1e-5, atol=1e-6) and torch.allclose(gw, rw, rtol=1e-4, atol=1e-5)


def test_weight_norm_and_pre_hook_of_the_layers():
    for layer in (slayer.synapse.Dense(6, 4, weight_norm=True), slayer.synapse.Conv(2, 3, 3, padding=1, weight_norm=True)):
        assert layer.weight_norm_enabled and hasattr(layer, 'weight_g')
        layer.disable_weight_norm()
        assert not layer.weight_norm_enabled and not hasattr(layer, 'weight_g')
        layer.pre_hook_fx = lambda w: w * 0
        x = torch.ones(1, 6, 4) if isinstance(layer, slayer.synapse.Dense) else torch.ones(1, 2, 4, 4, 5)
        assert float(layer(x).abs().max()) == 0.0


def test_pool_folds_the_channels_into_the_height_as_the_reference_does():
    gen = torch.Generator().manual_seed(6)
    pool = slayer.synapse.Pool(2, weight_scale=1.5)
    assert tuple(pool.weight.shape) == (1, 1, 2, 2, 1) and not pool.weight.requires_grad
    assert float(pool.weight.min()) == float(pool.weight.max()) == 1.5
    x = torch.randn(2, 3, 6, 8, 5, generator=gen)
    want = F.conv3d(x.reshape(2, 1, 18, 8, 5), 1.5 * torch.ones(1, 1, 2, 2, 1), None, (2, 2, 1)).reshape(2, 3, -1, 4, 5)
    assert torch.allclose(pool(x), want)
    # every output is the weighted sum of its own window of its own channel
    assert torch.allclose(pool(x)[1, 2, 1, 3], 1.5 * x[1, 2, 2:4, 6:8].sum(dim=(0, 1)))
    assert slayer.synapse.Pool((2, 3))(torch.randn(1, 2, 5, 7, 4, generator=gen)).shape == (1, 2, 3, 2, 4)
