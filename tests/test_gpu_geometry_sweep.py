"""Randomised geometry sweep of the streaming engine: many (rows, steps, alignment) combinations, each
checked by the independent one-thread-per-neuron kernels (debug=True raises on the first mismatch,
bit-exact for forward traces and input gradients).  The shapes are chosen to reach every kernel
variant: dword fallback (T % 4 != 0 or a misaligned view), the multi-wave kernel (few rows), the
one-wave kernel (more rows than fit the machine at once), partial last workgroups, rows that share
cache lines with their neighbours at every phase, rows shorter than a line."""
import numpy as np
import pytest
import torch

from tests.util import dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope='module')
def slayer():
    import lava_dl_amd.slayer as s
    return s


def _cases():
    rng = np.random.default_rng(20240607)
    cases = []
    for i in range(48):
        small = i % 3 != 2
        T = int(rng.choice([4, 8, 28, 32, 36, 60, 64, 68, 100, 124, 128, 132, 200, 300, 316, 37, 129, 1, 3]))
        if small:
            N, C, H = int(rng.integers(1, 5)), int(rng.integers(1, 40)), int(rng.integers(1, 30))
        else:                       # more rows than the multi-wave kernel takes: 140 K .. 300 K
            T = min(T, 64)
            N, C, H = int(rng.integers(2, 4)), int(rng.integers(300, 700)), int(rng.integers(100, 150))
        offset = int(rng.choice([0, 0, 4, 12, 20, 1, 2]))      # in floats: 16-byte aligned or not
        cases.append((N, C, H, T, offset))
    return cases


def _view(gen, shape, offset, scale=1.0, p=0.3):
    """A contiguous tensor that starts `offset` floats into its storage (changes the line phase)."""
    n = int(np.prod(shape))
    buf = torch.zeros(n + offset + 8)
    vals = (torch.rand(n, generator=gen) < p).float() * torch.randn(n, generator=gen) * scale
    buf[offset:offset + n] = vals
    return buf.to(dev())[offset:offset + n].view(shape)


@pytest.mark.parametrize('N,C,H,T,offset', _cases())
def test_li_and_res_against_the_independent_kernels(slayer, N, C, H, T, offset):
    gen = torch.Generator().manual_seed(N * 1000003 + C * 1009 + H * 101 + T * 7 + offset)
    shape = (N, C, H, T)
    D = slayer.neuron.dynamics
    x = _view(gen, shape, offset, 1.5).requires_grad_()
    x2 = _view(gen, shape, offset, 1.5).requires_grad_()
    g = _view(gen, shape, offset, 1.0, p=1.0)
    decay = torch.randint(0, 4097, (C,), generator=gen).float().to(dev()).requires_grad_()
    state = torch.randn(shape[:-1], generator=gen).to(dev())
    zero = torch.zeros(1, device=dev())
    y = D.leaky_integrator.dynamics(x, decay, state, 64, 1.0, debug=True)
    y.backward(g)
    assert x.grad is not None and torch.isfinite(x.grad).all()
    sin = (torch.rand(C, generator=gen) * 2000).round().to(dev()).requires_grad_()
    cos = (torch.rand(C, generator=gen) * 3000).round().to(dev()).requires_grad_()
    x.grad = None
    re, im = D.resonator.dynamics(x, x2, sin, cos, state, zero, 64, debug=True)
    (re * g + im).sum().backward()
    assert torch.isfinite(x.grad).all() and torch.isfinite(x2.grad).all()
    with torch.no_grad():
        D.adaptive_threshold.dynamics(x.detach(), zero, decay.detach(), zero + 1, decay.detach(), 0.5, 1.0, 64,
                                      debug=True)
        D.resonator.dynamics(x.detach(), x2.detach(), sin.detach(), cos.detach(), state, zero, 64, 0.8, debug=True)
