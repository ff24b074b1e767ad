"""Seeded sweep over geometries of the synapse kernels: convolution and transposed convolution (forward, input
gradient, weight gradient) with random kernel sizes, strides up to 16, paddings, dilations, channel counts (one
channel in and out takes the vector-unit kernel) and row lengths that are and are not whole quads, every element
against float64 evaluation of the reference's calls (synapse/layer.py:297-323, 630-658: F.conv3d / F.conv_transpose3d)
to 1e-5 of the sum of the magnitudes of its terms."""
import random

import pytest
import torch
import torch.nn.functional as F

from tests.util import assert_sum, dev

pytestmark = pytest.mark.gpu


def _geometry(rnd, wide):
    kh, kw = rnd.choice([1, 2, 3, 4, 5]), rnd.choice([1, 2, 3, 4, 5])
    if wide:
        sh, sw = rnd.choice([1, 2, 3, 4, 7, 16]), rnd.choice([1, 2, 3, 5, 8, 16])
    else:
        sh, sw = rnd.choice([1, 1, 2, 3, 4]), rnd.choice([1, 1, 2, 3, 5])
    dh, dw = rnd.choice([1, 1, 2, 3]), rnd.choice([1, 1, 2])
    ph, pw = rnd.randrange(0, 3), rnd.randrange(0, 3)
    ci, co = rnd.choice([1, 1, 2, 3, 8, 17]), rnd.choice([1, 1, 2, 5, 16, 20])
    n, t = rnd.choice([1, 2, 3]), rnd.choice([4, 7, 8, 36, 64, 65, 100])
    span = 40 if wide else 12
    h = rnd.randrange(dh * (kh - 1) + 1, dh * (kh - 1) + span)
    w = rnd.randrange(dw * (kw - 1) + 1, dw * (kw - 1) + span)
    return (n, ci, h, w, t), co, (kh, kw), (sh, sw), (ph, pw), (dh, dw)


@pytest.mark.parametrize('seed,wide,cases', [(1, False, 60), (2, False, 60), (7, True, 40)])
def test_sweep_of_convolution_geometries(seed, wide, cases):
    import lava_dl_amd.slayer as slayer
    rnd = random.Random(seed)
    gen = torch.Generator().manual_seed(rnd.randrange(1 << 30))
    for _ in range(cases):
        shape, co, kernel, stride, padding, dilation = _geometry(rnd, wide)
        what = f'{shape} -> {co}, kernel {kernel}, stride {stride}, padding {padding}, dilation {dilation}'
        cfg = (stride + (1,), padding + (0,), dilation + (1,))
        x = (torch.rand(shape, generator=gen) < 0.4).float() * torch.randn(shape, generator=gen)
        for transposed in (False, True):
            ci = shape[1]
            wt = torch.randn(*((ci, co) if transposed else (co, ci)), kernel[0], kernel[1], 1, generator=gen)
            if transposed:
                def reference(a, b):
                    return F.conv_transpose3d(a, b, None, cfg[0], cfg[1], 0, 1, cfg[2])
                if min((shape[2 + i] - 1) * stride[i] - 2 * padding[i] + dilation[i] * (kernel[i] - 1) + 1 for i in (0, 1)) < 1:
                    continue
                op = slayer.synapse.conv_transpose_synapse
            else:
                def reference(a, b):
                    return F.conv3d(a, b, None, *cfg)
                op = slayer.synapse.conv_synapse
            xg, wg = x.to(dev()).requires_grad_(), wt.to(dev()).requires_grad_()
            got = op(xg, wg, stride, padding, dilation)
            xd, wd = x.double().requires_grad_(), wt.double().requires_grad_()
            xa, wa = x.abs().double().requires_grad_(), wt.abs().double().requires_grad_()
            want, mag = reference(xd, wd), reference(xa, wa)
            name = ('transposed ' if transposed else '') + what
            assert got.shape == want.shape, name
            assert_sum(got, want.detach(), mag.detach() + 1e-30, name + ': forward')
            g = torch.randn(want.shape, generator=gen)
            got.backward(g.to(dev()))
            want.backward(g.double())
            mag.backward(g.abs().double())
            assert_sum(xg.grad, xd.grad, xa.grad + 1e-30, name + ': grad input')
            assert_sum(wg.grad, wd.grad, wa.grad + 1e-30, name + ': grad weight')
