"""Parity at the full benchmark sizes.  The oracle cannot run 10^8 neuron-timesteps in seconds, so each
configuration is checked two ways: (1) a subset of rows (neurons are independent) is recomputed by
the oracle and must match exactly; (2) a size-independent property over the whole tensor: splitting
the time axis and carrying the state must reproduce the single run bit for bit, and the backward
recurrences must be linear in the incoming gradient."""
import math

import pytest
import torch

from oracle import slayer_oracle as O
from tests.util import assert_exact, assert_rel, assert_same_gradient, assert_scale, assert_sum, dev, li_bwd_f64, SCAN_MIN

pytestmark = pytest.mark.gpu


@pytest.fixture(scope='module')
def slayer():
    import lava_dl_amd.slayer as s
    return s


def gpu_events(shape, p, amp, seed):
    g = torch.Generator(device=dev()).manual_seed(seed)
    return (torch.rand(shape, device=dev(), generator=g) < p).float() * \
        torch.randn(shape, device=dev(), generator=g) * amp


def gpu_randn(shape, seed):
    g = torch.Generator(device=dev()).manual_seed(seed)
    return torch.randn(shape, device=dev(), generator=g)


def test_cuba_conv_tensor_full_size(slayer):
    """config[1]: [32,16,32,32,300], per-channel decays, threshold 1.0, w_scale 64, fwd + bwd."""
    shape = (32, 16, 32, 32, 300)
    L = slayer.neuron.dynamics.leaky_integrator
    x = gpu_events(shape, 0.02, 0.5, 11)
    g = gpu_randn(shape, 12)
    gen = torch.Generator().manual_seed(13)
    d_i = torch.randint(0, 4096, (16,), generator=gen).float()
    d_v = torch.randint(0, 4096, (16,), generator=gen).float()
    zero = torch.zeros(1, device=dev())
    xg = x.clone().requires_grad_()
    dig, dvg = d_i.to(dev()).requires_grad_(), d_v.to(dev()).requires_grad_()
    cur = L.dynamics(xg, dig, zero, 64)
    vol = L.dynamics(cur, dvg, zero, 64, 1.0)
    spk = slayer.spike.Spike.apply(vol, 1.0, 1.0, 1.0, False, 0, 1)
    spk.backward(g)
    assert float(spk.detach().sum()) > 1000
    # (1) oracle on a slab: two batch entries, all channels, a corner of the image
    sl = (slice(None, None, 31), slice(None), slice(0, 32, 16), slice(0, 4))
    xs, gs = x[sl].cpu(), g[sl].cpu()
    r_cur = O.li_fwd(xs, d_i, torch.tensor([0.0]), 64)
    r_vol = O.li_fwd(r_cur, d_v, torch.tensor([0.0]), 64, 1.0)
    r_spk = O.spike_fwd(r_vol, 1.0)
    r_gv = O.spike_bwd(gs, r_vol, 1.0, 1.0, 1.0)
    r_gc, _ = O.li_bwd(r_gv, r_vol, d_v)
    r_gx, _ = O.li_bwd(r_gc, r_cur, d_i)
    assert_exact(cur[sl], r_cur, 'current slab')
    assert_exact(vol[sl], r_vol, 'voltage slab')
    assert_exact(spk[sl], r_spk, 'spike slab')
    assert_rel(xg.grad[sl], r_gx, 'grad_input slab')
    # parameter gradients: float64 sums of the GPU's own elementwise products
    g_vol = slayer.spike.spike._bwd(g, vol.detach(), None, 1.0, 1.0, 1.0, False)
    g_cur, _ = L._bwd(g_vol, vol.detach(), d_v.to(dev()), False)
    terms = g_cur[..., 1:].double() * vol.detach()[..., :-1].double()
    assert_sum(dvg.grad, terms.sum(dim=(0, 2, 3, 4)), terms.abs().sum(dim=(0, 2, 3, 4)), 'grad voltage_decay')
    del terms
    # (2) split invariance over the whole tensor
    k = 132
    c1 = L.dynamics(x[..., :k].contiguous(), d_i.to(dev()), zero, 64)
    v1 = L.dynamics(c1, d_v.to(dev()), zero, 64, 1.0)
    s1 = (v1[..., -1] >= 1.0).float()
    c2 = L.dynamics(x[..., k:].contiguous(), d_i.to(dev()), c1[..., -1].contiguous(), 64)
    v2 = L.dynamics(c2, d_v.to(dev()), L.persistent_state(v1[..., -1], s1).contiguous(), 64, 1.0)
    assert torch.equal(torch.cat([c1, c2], -1), cur.detach())
    assert torch.equal(torch.cat([v1, v2], -1), vol.detach())
    # linearity of the backward recurrence: bwd(2 g) == 2 bwd(g) exactly (power-of-two scaling)
    g2, _ = L._bwd(2 * g_vol, vol.detach(), d_v.to(dev()), False)
    assert torch.equal(g2, 2 * g_cur)


def test_alif_full_size(slayer):
    """config[2]: [64,512,1000], four per-channel decay vectors, th0 1.0, step 0.5."""
    shape = (64, 512, 1000)
    D = slayer.neuron.dynamics
    x = gpu_events(shape, 0.05, 1.0, 21)
    gen = torch.Generator().manual_seed(22)
    d = {k: torch.randint(0, 4096, (512,), generator=gen).float() for k in ('i', 'v', 'th', 'ref')}
    dg = {k: v.to(dev()) for k, v in d.items()}
    zero, one = torch.zeros(1, device=dev()), torch.ones(1, device=dev())
    cur = D.leaky_integrator.dynamics(x, dg['i'], zero, 64)
    vol = D.leaky_integrator.dynamics(cur, dg['v'], zero, 64)
    th, ref = D.adaptive_threshold.dynamics(vol, zero, dg['ref'], one, dg['th'], 0.5, 1.0, 64)
    spk = slayer.spike.Spike.apply(vol, th + ref, 1.0, 1.0, False, 0, 1)
    assert float(spk.detach().sum()) > 1000
    sl = (slice(None, None, 63), slice(None))            # first and last batch entry, all channels
    xs = x[sl].cpu()
    z1, o1 = torch.tensor([0.0]), torch.tensor([1.0])
    r_cur = O.li_fwd(xs, d['i'], z1, 64)
    r_vol = O.li_fwd(r_cur, d['v'], z1, 64)
    r_th, r_ref = O.ath_fwd(r_vol, z1, d['ref'], o1, d['th'], 0.5, 1.0, 64)
    assert_exact(vol[sl], r_vol, 'voltage')
    assert_exact(th[sl], r_th, 'threshold')
    assert_exact(ref[sl], r_ref, 'refractory')
    assert_exact(spk[sl], O.spike_fwd(r_vol, r_th + r_ref), 'spikes')
    # split invariance of the threshold / refractory pair with the persistent-state helpers
    k = 444
    A = D.adaptive_threshold
    t1, r1 = A.dynamics(vol[..., :k].contiguous(), zero, dg['ref'], one, dg['th'], 0.5, 1.0, 64)
    s1 = (vol[..., k - 1] >= t1[..., -1] + r1[..., -1]).float()
    t2, r2 = A.dynamics(vol[..., k:].contiguous(),
                        A.persistent_ref_state(r1[..., -1], s1, t1[..., -1]).contiguous(), dg['ref'],
                        A.persistent_th_state(t1[..., -1], s1, 0.5).contiguous(), dg['th'], 0.5, 1.0, 64)
    assert torch.equal(torch.cat([t1, t2], -1), th)
    assert torch.equal(torch.cat([r1, r2], -1), ref)
    del t1, t2, r1, r2
    # backward at full size (spike/spike.py:10-23, neuron/dynamics/leaky_integrator.py:234-259 in the reference):
    # surrogate against the tensor threshold, voltage recurrence, current recurrence -- by the three operators and
    # by the one fused kernel, both against the oracle on the slab, elementwise
    g = gpu_randn(shape, 23)
    theta = th + ref
    S = slayer.spike.spike
    g_vol = S._bwd(g, vol, theta, 0.0, 1.0, 1.0, False)
    g_cur, gd_v = D.leaky_integrator._bwd(g_vol, vol, dg['v'], True)
    g_x, gd_i = D.leaky_integrator._bwd(g_cur, cur, dg['i'], True)
    f_x, f_gi, f_gv = D.alif_fused._bwd(g, vol, theta, cur, dg['i'], dg['v'], 1.0, 1.0, False, True)
    assert torch.equal(f_x, g_x), 'fused ALIF backward differs from the operator chain'
    gs = g[sl].cpu()
    o_gv = O.spike_bwd(gs, r_vol, r_th + r_ref, 1.0, 1.0)
    o_gc, _ = O.li_bwd(o_gv, r_vol, d['v'])
    o_gx, _ = O.li_bwd(o_gc, r_cur, d['i'])
    assert_rel(g_vol[sl], o_gv, 'spike surrogate slab')
    assert_scale(g_cur[sl], o_gc, 'voltage gradient slab')
    assert_scale(g_x[sl], o_gx, 'input gradient slab')
    # element by element: each recurrence in float64 on the very gradient the kernel read, against the sum of the
    # magnitudes of the terms that make up the element
    T = shape[-1]
    for name, got, fed, dec in (('voltage', g_cur, g_vol, d['v']), ('input', g_x, g_cur, d['i'])):
        a = (1 - dec / 4096).repeat(2)                   # rows of the slab: 2 batch entries x 512 channels
        want, mag = li_bwd_f64(fed[sl].reshape(-1, T), a)
        assert_sum(got[sl].reshape(-1, T), want, mag, f'{name} gradient slab, elementwise')
    # decay gradients: float64 sums of the GPU's own products, held to 1e-5 of the sum of the terms' magnitudes
    for name, got, fused, grad_next, trace in (('voltage', gd_v, f_gv, g_cur, vol), ('current', gd_i, f_gi, g_x, cur)):
        terms = grad_next[..., 1:].double() * trace[..., :-1].double()
        want, mag = terms.sum(dim=(0, 2)), terms.abs().sum(dim=(0, 2))
        assert_sum(got, want, mag, f'grad {name} decay')
        assert_sum(fused, want, mag, f'fused grad {name} decay')


def test_rf_full_size(slayer):
    """config[3]: [64,1024,2000] real/imag pair, per-channel rotation, phase-threshold spike, fwd + bwd."""
    shape = (64, 1024, 2000)
    R = slayer.neuron.dynamics.resonator
    xr, xi = gpu_events(shape, 0.1, 0.3, 31), gpu_events(shape, 0.1, 0.3, 32)
    gen = torch.Generator().manual_seed(33)
    decay = torch.randint(0, 4096, (1024,), generator=gen).float()
    phi = 2 * math.pi * (5 + 45 * torch.rand(1024, generator=gen)) * 1e-3
    sin = ((4096 - decay) * torch.sin(phi)).round().clamp_min(1)
    cos = ((4096 - decay) * torch.cos(phi)).round().clamp_min(0)
    zero = torch.zeros(1, device=dev())
    sg, cg = sin.to(dev()), cos.to(dev())
    re, im = R.dynamics(xr, xi, sg, cg, zero, zero, 64)
    spk = slayer.spike.complex.Spike.apply(re, im, 1.0, 0.5, 10.0, False, 0, 1)
    assert float(spk.detach().sum()) > 1000
    sl = (slice(None, None, 63), slice(None, None, 8))      # 2 batch entries x 128 channels
    z1 = torch.tensor([0.0])
    r_re, r_im = O.res_fwd(xr[sl].cpu(), xi[sl].cpu(), sin[::8], cos[::8], z1, z1, 64)
    assert_exact(re[sl], r_re, 'real')
    assert_exact(im[sl], r_im, 'imag')
    assert_exact(spk[sl], O.cspike_fwd(r_re, r_im, 1.0, 0.0), 'spikes')
    del spk
    g = gpu_randn(shape, 34)
    from lava_dl_amd.slayer.spike import complex as CS
    g_re, g_im = CS._bwd(g, re, im, None, 1.0, 0.5, 10.0, False)
    w_re, w_im = O.cspike_bwd(g[sl].cpu(), r_re, r_im, 1.0, 0.5, 10.0)
    assert_rel(g_re[sl], w_re, 'cspike grad real')
    assert_rel(g_im[sl], w_im, 'cspike grad imag')
    gr, gi, gs, gc = R._bwd(g_re, g_im, re, im, sg, cg)
    w = O.res_bwd(g_re[sl].cpu(), g_im[sl].cpu(), r_re, r_im, sin[::8], cos[::8])
    assert_scale(gr[sl], w[0], 'res_bwd grad real')
    assert_scale(gi[sl], w[1], 'res_bwd grad imag')
    assert torch.isfinite(gs).all() and torch.isfinite(gc).all()
    # split invariance
    k = 1036
    a_re, a_im = R.dynamics(xr[..., :k].contiguous(), xi[..., :k].contiguous(), sg, cg, zero, zero, 64)
    b_re, b_im = R.dynamics(xr[..., k:].contiguous(), xi[..., k:].contiguous(), sg, cg,
                            a_re[..., -1].contiguous(), a_im[..., -1].contiguous(), 64)
    assert torch.equal(torch.cat([a_re, b_re], -1), re)
    assert torch.equal(torch.cat([a_im, b_im], -1), im)


def test_synapse_stack_full_size(slayer):
    """config[4]: conv (K=64 alpha kernel) -> per-channel shift -> CUBA on [32,256,1500], fwd + bwd."""
    shape = (32, 256, 1500)
    gen = torch.Generator(device=dev()).manual_seed(41)
    x = (torch.rand(shape, device=dev(), generator=gen) < 0.03).float()
    i = torch.arange(64, dtype=torch.float32)
    filt = (i / 4) * torch.exp(1 - i / 4)
    delay = torch.rand(256, generator=torch.Generator().manual_seed(42)) * 32
    L = slayer.neuron.dynamics.leaky_integrator
    zero = torch.zeros(1, device=dev())
    d_i, d_v = torch.tensor([1024.0]), torch.tensor([128.0])
    xg = x.clone().requires_grad_()
    y = slayer.utils.filter.conv(xg, filt.to(dev()), 1)
    axon = slayer.axon.Delay()
    axon.delay.data, axon.init = delay.to(dev()), True
    z = axon(y)
    cur = L.dynamics(z, d_i.to(dev()), zero, 64)
    vol = L.dynamics(cur, d_v.to(dev()), zero, 64, 1.25)
    spk = slayer.spike.Spike.apply(vol, 1.25, 1.0, 1.0, False, 0, 1)
    g = gpu_randn(shape, 43)
    spk.backward(g)
    assert float(spk.detach().sum()) > 1000
    sl = (slice(None, None, 31),)
    xs = x[sl].cpu()
    r_y = O.conv_fwd(xs, filt, 1)
    assert_rel(y[sl], r_y, 'conv')
    # downstream stages are checked on the GPU's own conv output so that float rounding of the filter
    # sum cannot flip an integer truncation
    ys = y[sl].detach().cpu()
    r_z = O.shift(ys, delay, 1)
    assert_exact(z[sl], r_z, 'shift')
    z1 = torch.tensor([0.0])
    r_cur = O.li_fwd(r_z, d_i, z1, 64)
    r_vol = O.li_fwd(r_cur, d_v, z1, 64, 1.25)
    assert_exact(vol[sl], r_vol, 'voltage')
    assert_exact(spk[sl], O.spike_fwd(r_vol, 1.25), 'spikes')
    r_gv = O.spike_bwd(g[sl].cpu(), r_vol, 1.25, 1.0, 1.0)
    r_gc, _ = O.li_bwd(r_gv, r_vol, d_v)
    r_gz, _ = O.li_bwd(r_gc, r_cur, d_i)
    r_gx = O.conv_bwd(O.shift(r_gz, -delay, 1), filt, 1)
    assert_scale(xg.grad[sl], r_gx, 'grad through the stack')
    # adjointness <conv(x), g> == <x, corr(g)> over the whole tensor, in float64.  Both sides are sums of 12 M terms
    # of either sign that cancel to about 1e-5 of the sum of their magnitudes; every output carries a float32
    # rounding error of up to 1e-7 of its value, and the matrix instructions round toward zero on the way (a bias of
    # about 1e-8 that does not average out), so the bar is 1e-8 of the sum of the magnitudes.  A tap or a step off by
    # one moves the two sides apart by more than that sum's thousandth.
    lhs = (y.detach().double() * g.double()).sum()
    rhs = (x.double() * slayer.utils.filter.corr(g, filt.to(dev()), 1).double()).sum()
    magnitudes = float((y.detach().double().abs() * g.double().abs()).sum())
    assert abs(float(lhs - rhs)) <= 1e-8 * magnitudes


@pytest.mark.parametrize('C,T', [(300000, 1000), (150000, 999)])
def test_tensors_beyond_four_gib(slayer, C, T):
    """[8, 300000, 1000] float32 is 9.6 GB per tensor (dwordx4 kernels), [8, 150000, 999] 4.8 GB (dword
    kernels): byte offsets pass 2**32 and, in the first, element offsets pass 2**31 inside the tensor.  Row
    slabs at the start, around those two lines and at the end are recomputed by the oracle; the fused CUBA
    block must equal the chain everywhere."""
    N = 8
    shape = (N, C, T)
    D = slayer.neuron.dynamics
    L = D.leaky_integrator
    x = gpu_events(shape, 0.03, 0.6, 31 + T)
    g = gpu_randn(shape, 32 + T)
    d_i, d_v = torch.tensor([1024.0]), torch.tensor([128.0])
    zero = torch.zeros(1, device=dev())
    cur = L.dynamics(x, d_i.to(dev()), zero, 64)
    vol = L.dynamics(cur, d_v.to(dev()), zero, 64, 1.25)
    spk = slayer.spike.spike._fwd(vol, None, 1.25, False, 1.0)
    g_vol = slayer.spike.spike._bwd(g, vol, None, 1.25, 1.0, 1.0, False)
    g_cur, _ = L._bwd(g_vol, vol, d_v.to(dev()), False)
    slabs = [(0, slice(0, 70)), (N - 1, slice(C - 70, C))]
    for line in (1 << 30, 1 << 31):                 # element index of byte 2**32 and element 2**31
        if line < N * C * T:
            n0, c0 = divmod(line // T, C)
            slabs.append((n0, slice(max(c0 - 40, 0), min(c0 + 40, C))))
    for n, cs in slabs:
        xs, gs = x[n:n + 1, cs].cpu(), g[n:n + 1, cs].cpu()
        r_cur = O.li_fwd(xs, d_i, torch.tensor([0.0]), 64)
        r_vol = O.li_fwd(r_cur, d_v, torch.tensor([0.0]), 64, 1.25)
        r_spk = O.spike_fwd(r_vol, 1.25)
        r_gv = O.spike_bwd(gs, r_vol, 1.25, 1.0, 1.0)
        r_gc, _ = O.li_bwd(g_vol[n:n + 1, cs].cpu(), r_vol, d_v)     # the GPU's own surrogate values: exact compare
        assert_exact(cur[n:n + 1, cs], r_cur, f'current slab {n} T={T}')
        assert_exact(vol[n:n + 1, cs], r_vol, f'voltage slab {n} T={T}')
        assert_exact(spk[n:n + 1, cs], r_spk, f'spike slab {n} T={T}')
        assert_rel(g_vol[n:n + 1, cs], r_gv, f'spike grad slab {n} T={T}')
        assert_scale(g_cur[n:n + 1, cs], r_gc, f'li_bwd slab {n} T={T}')
    assert float(spk.sum()) > 1000
    del g, g_vol, g_cur
    f_cur, f_vol, f_spk = D.cuba_fused._fwd(x, d_i.to(dev()), d_v.to(dev()), zero, zero, 64, 1.25, False, 1.0)[:3]
    assert torch.equal(f_cur, cur) and torch.equal(f_vol, vol) and torch.equal(f_spk, spk)
    del f_cur, f_vol, f_spk, cur, vol, spk, x
    torch.cuda.empty_cache()


@pytest.mark.parametrize('T', [512, 1024, 500])
def test_rows_a_power_of_two_apart_take_long_pieces_with_the_same_results(slayer, T):
    """Tensors too large for the all-resident kernel whose rows are (nearly) a multiple of 2 KB apart: LI forward
    and the fused CUBA forward switch to 16 rows per wave there.  Oracle on a slab of rows, the fused kernel against
    the chain of operators over the whole tensor, and the split-in-time invariance."""
    M0 = 160 * 1024 * 1024 // T                        # 640 MB per tensor: far more rows than stay resident
    shape = (M0 // 64, 64, T)
    D = slayer.neuron.dynamics
    L = D.leaky_integrator
    x = gpu_events(shape, 0.05, 1.0, 70 + T)
    gen = torch.Generator().manual_seed(71)
    d_i = torch.randint(0, 4096, (64,), generator=gen).float()
    d_v = torch.randint(0, 4096, (64,), generator=gen).float()
    zero = torch.zeros(1, device=dev())
    cur = L._fwd(x, d_i.to(dev()), zero, -1, 4096)
    vol = L._fwd(cur, d_v.to(dev()), zero, 1.25, 4096)
    f_cur, f_vol, f_spk = D.cuba_fused._fwd(x, d_i.to(dev()), d_v.to(dev()), zero, zero, 4096, 1.25, False, 1)
    assert torch.equal(f_cur, cur) and torch.equal(f_vol, vol)
    assert torch.equal(f_spk, (vol >= 1.25).float()) and float(f_spk.sum()) > 1000
    sl = (slice(None, None, shape[0] // 3), slice(None, None, 7))
    r_cur = O.li_fwd(x[sl].cpu(), d_i[::7], torch.tensor([0.0]), 4096)
    r_vol = O.li_fwd(r_cur, d_v[::7], torch.tensor([0.0]), 4096, 1.25)
    assert_exact(cur[sl], r_cur, 'current slab')
    assert_exact(vol[sl], r_vol, 'voltage slab')
    k = T // 2 + 4
    c1 = L._fwd(x[..., :k].contiguous(), d_i.to(dev()), zero, -1, 4096)
    c2 = L._fwd(x[..., k:].contiguous(), d_i.to(dev()), c1[..., -1].contiguous(), -1, 4096)
    assert torch.equal(torch.cat([c1, c2], -1), cur)
