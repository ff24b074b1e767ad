"""Randomised geometry sweep of the streaming engine: many (rows, steps, alignment) combinations, each
checked by the independent one-thread-per-neuron kernels (debug=True raises on the first mismatch,
bit-exact for forward traces and input gradients).  The shapes are chosen to reach every kernel
variant: dword fallback (T % 4 != 0 or a misaligned view), the multi-wave kernel (few rows), the
one-wave kernel (more rows than fit the machine at once), partial last workgroups, rows that share
cache lines with their neighbours at every phase, rows shorter than a line."""
import numpy as np
import pytest
import torch

from tests.util import assert_same_gradient, assert_scale, dev, SCAN_MIN

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


# Rows that are not whole quads (T % 4 != 0) or that start at addresses that are only dword-aligned: the multi-wave
# kernels' form for them (csrc/tile.h, UNAL), where a row may begin and end inside a 16-byte quad.
def _unaligned_cases():
    rng = np.random.default_rng(4242)
    cases = []
    # rows of 256 steps and more take the multi-wave form, shorter ones the dword kernel
    for T in [5, 6, 7, 9, 13, 30, 31, 33, 34, 35, 61, 63, 65, 66, 95, 97, 127, 130, 131, 255, 257, 258, 259, 261, 287, 289,
              301, 302, 303, 319, 321, 350, 450, 1001]:
        N, C, H = int(rng.integers(1, 4)), int(rng.integers(1, 40)), int(rng.integers(1, 12))
        cases.append((N, C, H, T, int(rng.integers(0, 4))))
    for T, offset in [(256, 1), (300, 2), (320, 3), (1000, 1)]:       # whole quads in length, dword-aligned start
        cases.append((2, int(rng.integers(1, 40)), int(rng.integers(1, 12)), T, offset))
    cases.append((2, 600, 130, 37, 1))      # more workgroups than the chip holds at once: dword kernel
    cases.append((2, 300, 130, 257, 1))     # ... multi-wave form
    cases.append((3, 400, 110, 64, 3))
    return cases


@pytest.mark.parametrize('N,C,H,T,offset', _unaligned_cases())
def test_rows_that_are_not_whole_quads(slayer, N, C, H, T, offset):
    test_li_and_res_against_the_independent_kernels(slayer, N, C, H, T, offset)


@pytest.mark.parametrize('N,C,H,T,offset', _unaligned_cases()[::3])
@pytest.mark.parametrize('graded', [False, True])
def test_fused_blocks_on_rows_that_are_not_whole_quads(slayer, N, C, H, T, offset, graded):
    test_fused_blocks_against_the_operator_chains(slayer, N, C, H, T, offset, 64, graded)


def _fused_cases():
    rng = np.random.default_rng(977)
    cases = []
    for i in range(30):
        big = i % 5 == 4
        T = int(rng.choice([4, 8, 28, 32, 36, 60, 64, 100, 124, 128, 132, 200, 300, 316, 1000, 37, 129, 3]))
        if big:                     # more rows than the multi-wave kernels take
            T = min(T, 36)
            N, C, H = int(rng.integers(2, 4)), int(rng.integers(300, 700)), int(rng.integers(100, 150))
        else:
            N, C, H = int(rng.integers(1, 5)), int(rng.integers(1, 40)), int(rng.integers(1, 30))
        offset = int(rng.choice([0, 0, 4, 12, 20, 1]))
        w = int(rng.choice([64, 64, 4096, 100]))
        graded = bool(rng.integers(0, 2))
        cases.append((N, C, H, T, offset, w, graded))
    return cases


@pytest.mark.parametrize('N,C,H,T,offset,w,graded', _fused_cases())
def test_fused_blocks_against_the_operator_chains(slayer, N, C, H, T, offset, w, graded):
    """Fused CUBA / ALIF / RF kernels (integer tiles, surrogate staged by one to four copy waves, three- and
    four-tile forms) against the chains of stand-alone operators over random geometries: traces, spikes and input
    gradients bit for bit, with and without decay gradients."""
    gen = torch.Generator().manual_seed(N * 1000003 + C * 1009 + H * 101 + T * 7 + offset + w)
    shape = (N, C, H, T)
    D = slayer.neuron.dynamics
    Spike, CSpike = slayer.spike.Spike, slayer.spike.complex.Spike
    x = _view(gen, shape, offset, 1.5)
    x2 = _view(gen, shape, offset, 1.5)
    g = _view(gen, shape, offset, 1.0, p=1.0)
    dec = [torch.randint(0, 4097, (C,), generator=gen).float().to(dev()) for _ in range(4)]
    st = [torch.randn(shape[:-1], generator=gen).to(dev()) for _ in range(3)]
    thr, tau, rho, scale = 0.75, 0.8, 1.2, 2

    def grads(fn, inputs, params):
        """(outputs, input grads, parameter grads) of fn on fresh leaves."""
        xs = [t.clone().requires_grad_() for t in inputs]
        ps = [t.clone().requires_grad_() for t in params]
        outs = fn(xs, ps)
        outs[-1].backward(g)
        return [o.detach() for o in outs], [t.grad for t in xs], [t.grad for t in ps]

    # ---- CUBA
    def cuba_chain(xs, ps):
        cur = D.leaky_integrator.dynamics(xs[0], ps[0], st[0], w)
        vol = D.leaky_integrator.dynamics(cur, ps[1], st[1], w, thr)
        return [cur, vol, Spike.apply(vol, thr, tau, rho, graded, 0, scale)]
    ref_o, ref_gx, ref_gp = grads(cuba_chain, [x], dec[:2])
    got_o, got_gx, got_gp = grads(lambda xs, ps: list(D.cuba_fused.dynamics(
        xs[0], ps[0], ps[1], st[0], st[1], w, thr, tau, rho, graded, scale)), [x], dec[:2])
    assert all(torch.equal(a, b) for a, b in zip(got_o, ref_o)), 'CUBA outputs'
    assert_same_gradient(got_gx[0], ref_gx[0], 'CUBA grad input')
    for a, b in zip(got_gp, ref_gp):
        assert torch.allclose(a, b, rtol=1e-5, atol=1e-5 * float(b.abs().max())), 'CUBA decay grads'
    xl = x.clone().requires_grad_()
    lean = D.cuba_fused.dynamics(xl, dec[0], dec[1], st[0], st[1], w, thr, tau, rho, graded, scale, keep_current=False)
    lean[2].backward(g)
    assert torch.equal(lean[2].detach(), ref_o[2]), 'CUBA lean'
    assert_same_gradient(xl.grad, ref_gx[0], 'CUBA lean grad input')

    # ---- ALIF
    th0 = (1.0 + torch.rand(shape[:-1], generator=gen)).to(dev())

    def alif_chain(xs, ps):
        cur = D.leaky_integrator.dynamics(xs[0], ps[0], st[0], w)
        vol = D.leaky_integrator.dynamics(cur, ps[1], st[1], w)
        th, ref = D.adaptive_threshold.dynamics(vol, st[2].abs(), dec[3], th0, dec[2], 0.5, 1.0, w)
        return [cur, vol, th + ref, Spike.apply(vol, th + ref, tau, rho, graded, 0, scale)]
    ref_o, ref_gx, ref_gp = grads(alif_chain, [x], dec[:2])
    got_o, got_gx, got_gp = grads(lambda xs, ps: list(D.alif_fused.dynamics(
        xs[0], ps[0], ps[1], dec[2], dec[3], st[0], st[1], th0, st[2].abs(), 0.5, 1.0, w, tau, rho, graded, scale)[:4]),
        [x], dec[:2])
    assert all(torch.equal(a, b) for a, b in zip(got_o, ref_o)), 'ALIF outputs'
    assert_same_gradient(got_gx[0], ref_gx[0], 'ALIF grad input')
    xl = x.clone().requires_grad_()
    lean = D.alif_fused.dynamics(xl, dec[0], dec[1], dec[2], dec[3], st[0], st[1], th0, st[2].abs(), 0.5, 1.0, w,
                                 tau, rho, graded, scale, keep_current=False)
    lean[3].backward(g)
    assert torch.equal(lean[3].detach(), ref_o[3]), 'ALIF lean'
    assert_same_gradient(xl.grad, ref_gx[0], 'ALIF lean grad input')

    # ---- RF
    sin = (torch.rand(C, generator=gen) * 2000).round().to(dev())
    cos = (torch.rand(C, generator=gen) * 3000).round().to(dev())
    last = st[2]

    def rf_chain(xs, ps):
        re, im = D.resonator.dynamics(xs[0], xs[1], ps[0], ps[1], st[0], st[1], w)
        return [re, im, CSpike.apply(re, im, thr, tau, rho, graded, last, scale)]
    ref_o, ref_gx, ref_gp = grads(rf_chain, [x, x2], [sin, cos])
    got_o, got_gx, got_gp = grads(lambda xs, ps: list(D.rf_fused.dynamics(
        xs[0], xs[1], ps[0], ps[1], st[0], st[1], last, w, thr, tau, rho, graded, scale)), [x, x2], [sin, cos])
    assert all(torch.equal(a, b) for a, b in zip(got_o, ref_o)), 'RF outputs'
    assert_same_gradient(got_gx[0], ref_gx[0], 'RF grad real input')
    assert_same_gradient(got_gx[1], ref_gx[1], 'RF grad imag input')
    for a, b in zip(got_gp, ref_gp):
        assert torch.allclose(a, b, rtol=1e-5, atol=1e-5 * float(b.abs().max())), 'RF decay grads'
    xl, xl2 = x.clone().requires_grad_(), x2.clone().requires_grad_()
    lean = D.rf_fused.dynamics(xl, xl2, sin, cos, st[0], st[1], last, w, thr, tau, rho, graded, scale)
    lean[2].backward(g)
    assert torch.equal(lean[2].detach(), ref_o[2]), 'RF lean spikes'
    assert_same_gradient(xl.grad, ref_gx[0], 'RF lean grad real')
    assert_same_gradient(xl2.grad, ref_gx[1], 'RF lean grad imag')
