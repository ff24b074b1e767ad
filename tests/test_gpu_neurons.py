"""The thin CUBA / ALIF / RF neuron modules against the oracle's op chain, plus the invariants the
reference's neuron tests assert (tests/lava/lib/dl/slayer/neuron/test_cuba.py:91-271 and siblings):
batch consistency, integer states, persistent-state split invariance, backward runs."""
import numpy as np
import pytest
import torch

from oracle import slayer_oracle as O
from tests.util import assert_exact, assert_rel, assert_same_gradient, assert_scale, dev, sparse_input, SCAN_MIN

pytestmark = pytest.mark.gpu


@pytest.fixture(scope='module')
def slayer():
    import lava_dl_amd.slayer as s
    return s


def _oracle_cuba(x, cd, vd, thr, s_scale, tau, rho, cs=None, vs=None):
    zero = torch.tensor([0.0])
    cur = O.li_fwd(x, cd, zero if cs is None else cs, s_scale)
    vol = O.li_fwd(cur, vd, zero if vs is None else vs, s_scale, thr)
    return cur, vol, O.spike_fwd(vol, thr)


def test_cuba_neuron_matches_oracle_chain(slayer):
    gen = torch.Generator().manual_seed(100)
    x = sparse_input(gen, (2, 6, 5, 80), p=0.2, amp=1.0)
    n = slayer.neuron.cuba.Neuron(threshold=1.0, current_decay=0.25, voltage_decay=0.03,
                                  tau_grad=1, scale_grad=1, requires_grad=True).to(dev())
    xg = x.to(dev()).requires_grad_()
    cur, vol = n.dynamics(xg)
    spk = n.spike(vol)
    thr = 1.0 + 0.01 / 4096
    cd, vd = torch.tensor([1024.0]), torch.tensor([round(0.03 * 4096) * 1.0])
    r_cur, r_vol, r_spk = _oracle_cuba(x, cd, vd, thr, 4096, 100.0, 0.1)
    assert_exact(cur, r_cur, 'cuba current')
    assert_exact(vol, r_vol, 'cuba voltage')
    assert_exact(spk, r_spk, 'cuba spikes')
    assert r_spk.sum() > 0
    g = torch.randn(x.shape, generator=gen)
    spk.backward(g.to(dev()))
    r_gv = O.spike_bwd(g, r_vol, thr, 1.0 * 100, 1 * 0.1)
    r_gc, r_gvd = O.li_bwd(r_gv, r_vol, vd)
    r_gx, r_gcd = O.li_bwd(r_gc, r_cur, cd)
    assert_rel(xg.grad, r_gx, 'cuba grad_input')
    assert_rel(n.voltage_decay.grad, r_gvd, 'cuba grad voltage_decay')
    assert_rel(n.current_decay.grad, r_gcd, 'cuba grad current_decay')
    # integer states at the state scale, identical batch entries give identical outputs
    assert torch.equal(torch.floor(vol * 4096), vol * 4096)
    xb = x[:1].repeat(3, 1, 1, 1).to(dev())
    n2 = slayer.neuron.cuba.Neuron(1.0, 0.25, 0.03).to(dev())
    assert float(n2(xb).var(dim=0).max()) == 0.0


@pytest.mark.parametrize('kind', ['cuba', 'alif', 'rf'])
@pytest.mark.parametrize('shared', [True, False])
def test_persistent_state_split_invariance(slayer, kind, shared):
    """Running [:k] then [k:] with carried state equals the full run, for every trace and the spikes."""
    gen = torch.Generator().manual_seed(101)
    shape, k = (3, 8, 120), 47
    torch.manual_seed(5)
    if kind == 'cuba':
        mk = lambda p: slayer.neuron.cuba.Neuron(1.0, [0.2, 0.4] if not shared else 0.25,
                                                 [0.02, 0.2] if not shared else 0.03,
                                                 shared_param=shared, persistent_state=p).to(dev())
        x = sparse_input(gen, shape, p=0.3).to(dev())
        run = lambda n, inp: (lambda cv: (cv[0], cv[1], n.spike(cv[1])))(n.dynamics(inp))
    elif kind == 'alif':
        rng = lambda a, b: [a, b] if not shared else a
        mk = lambda p: slayer.neuron.alif.Neuron(1.0, 0.5, rng(0.25, 0.4), rng(0.03, 0.2), rng(0.1, 0.3),
                                                 rng(0.1, 0.3), shared_param=shared, persistent_state=p).to(dev())
        x = sparse_input(gen, shape, p=0.4, amp=2.0).to(dev())
        run = lambda n, inp: (lambda t: t + (n.spike(t[1], t[2], t[3]),))(n.dynamics(inp))
    else:
        mk = lambda p: slayer.neuron.rf.Neuron(1.0, [5, 20] if not shared else 11,
                                               [0.02, 0.1] if not shared else 0.05,
                                               shared_param=shared, persistent_state=p).to(dev())
        x = (sparse_input(gen, shape, p=0.3).to(dev()), sparse_input(gen, shape, p=0.3).to(dev()))
        run = lambda n, inp: (lambda t: t + (n.spike(t[0], t[1]),))(n.dynamics(inp))
    cut = (lambda a, b: tuple(t[..., a:b] for t in x)) if kind == 'rf' else (lambda a, b: x[..., a:b])
    full_n, split_n = mk(False), mk(True)
    full = run(full_n, x)
    # same parameters in both modules
    split_n._prepare(x[0] if kind == 'rf' else x)
    for (na, pa), (nb, pb) in zip(full_n.named_parameters(), split_n.named_parameters()):
        pb.data = pa.data.clone()
    a = run(split_n, cut(0, k))
    b = run(split_n, cut(k, shape[-1]))
    assert sum(float(t.sum()) for t in (full[-1],)) > 0, 'no spikes in the test workload'
    for i, (f, pa, pb) in enumerate(zip(full, a, b)):
        assert torch.equal(torch.cat([pa, pb], dim=-1), f), f'{kind} trace {i} differs after the split'


def test_alif_neuron_matches_oracle_chain(slayer):
    gen = torch.Generator().manual_seed(102)
    x = sparse_input(gen, (2, 12, 150), p=0.4, amp=2.0)
    n = slayer.neuron.alif.Neuron(threshold=1.0, threshold_step=0.5, current_decay=0.25, voltage_decay=0.1,
                                  threshold_decay=0.05, refractory_decay=0.2).to(dev())
    xg = x.to(dev()).requires_grad_()
    cur, vol, th, ref = n.dynamics(xg)
    spk = n.spike(vol, th, ref)
    one, zero = torch.tensor([1.0]), torch.tensor([0.0])
    q = lambda v: torch.tensor([float(round(v * 4096))])
    r_cur = O.li_fwd(x, q(0.25), zero, 4096)
    r_vol = O.li_fwd(r_cur, q(0.1), zero, 4096)
    r_th, r_ref = O.ath_fwd(r_vol, zero, q(0.2), one, q(0.05), 0.5, 1.0, 4096)
    r_spk = O.spike_fwd(r_vol, r_th + r_ref)
    for got, ref_t, name in ((cur, r_cur, 'current'), (vol, r_vol, 'voltage'), (th, r_th, 'threshold'),
                             (ref, r_ref, 'refractory'), (spk, r_spk, 'spikes')):
        assert_exact(got, ref_t, f'alif {name}')
    assert r_spk.sum() > 0
    g = torch.randn(x.shape, generator=gen)
    spk.backward(g.to(dev()))
    r_gv = O.spike_bwd(g, r_vol, r_th + r_ref, 100.0, 0.1)
    r_gc, _ = O.li_bwd(r_gv, r_vol, q(0.1))
    r_gx, _ = O.li_bwd(r_gc, r_cur, q(0.25))
    assert_rel(xg.grad, r_gx, 'alif grad_input')


def test_rf_neuron_matches_oracle_chain(slayer):
    gen = torch.Generator().manual_seed(103)
    shape = (2, 10, 200)
    xr, xi = sparse_input(gen, shape, p=0.3), sparse_input(gen, shape, p=0.3)
    n = slayer.neuron.rf.Neuron(threshold=1.0, period=11, decay=0.05).to(dev())
    rg, ig = xr.to(dev()).requires_grad_(), xi.to(dev()).requires_grad_()
    re, im = n.dynamics((rg, ig))
    spk = n.spike(re, im)
    sin = torch.round(n.sin_decay.detach().cpu())
    cos = torch.round(n.cos_decay.detach().cpu())
    assert (sin.item(), cos.item()) == (2104.0, 3273.0)
    zero = torch.tensor([0.0])
    r_re, r_im = O.res_fwd(xr, xi, sin, cos, zero, zero, 4096)
    r_spk = O.cspike_fwd(r_re, r_im, 1.0, 0.0)
    assert_exact(re, r_re, 'rf real')
    assert_exact(im, r_im, 'rf imag')
    assert_exact(spk, r_spk, 'rf spikes')
    assert r_spk.sum() > 0
    g = torch.randn(shape, generator=gen)
    spk.backward(g.to(dev()))
    g_re, g_im = O.cspike_bwd(g, r_re, r_im, 1.0, 0.5, 10.0)
    r_gr, r_gi, _, _ = O.res_bwd(g_re, g_im, r_re, r_im, sin, cos)
    assert_rel(rg.grad, r_gr, 'rf grad real input')
    assert_rel(ig.grad, r_gi, 'rf grad imag input')


def test_neuron_shape_checks(slayer):
    n = slayer.neuron.cuba.Neuron(1.0, 0.25, 0.03).to(dev())
    with pytest.raises(AssertionError):
        n(torch.zeros(4, 10, device=dev()))
    n(torch.zeros(2, 3, 10, device=dev()))
    with pytest.raises(AssertionError):
        n(torch.zeros(2, 4, 10, device=dev()))
    with pytest.raises(AssertionError):
        slayer.neuron.cuba.Neuron(1.0, [0.1, 0.2], 0.03)
    with pytest.raises(AssertionError):
        slayer.neuron.rf.Neuron(1.0, 3, 0.05)


@pytest.mark.parametrize('shape,w,graded', [((4, 16, 8, 8, 300), 64, False), ((3, 70, 129), 100, False),
                                            ((2, 3, 5, 7, 37), 4096, True), ((4, 9000, 64), 64, False),
                                            ((4, 70000, 40), 64, False)])
def test_fused_cuba_equals_the_operator_chain(slayer, shape, w, graded):
    """The fused kernels must reproduce leaky_integrator -> leaky_integrator(threshold) -> Spike bit for bit,
    forward (all three traces) and backward (grad_input), and the decay gradients to float tolerance."""
    from tests.util import seed_of
    gen = torch.Generator().manual_seed(seed_of(shape, w, graded, 'fused'))
    C = shape[1]
    x = sparse_input(gen, shape, p=0.1, amp=1.5).to(dev())
    g = torch.randn(shape, generator=gen).to(dev())
    d_i = torch.randint(0, 4097, (C,), generator=gen).float().to(dev())
    d_v = torch.randint(0, 4097, (C,), generator=gen).float().to(dev())
    s_i = torch.randn(shape[:-1], generator=gen).to(dev())
    s_v = torch.randn(shape[:-1], generator=gen).to(dev()) * 0.3
    thr, tau, rho = 1.0 + 0.01 / w, 1.3, 0.7
    D = slayer.neuron.dynamics
    # chain
    x1, di1, dv1 = x.clone().requires_grad_(), d_i.clone().requires_grad_(), d_v.clone().requires_grad_()
    cur = D.leaky_integrator.dynamics(x1, di1, s_i, w)
    vol = D.leaky_integrator.dynamics(cur, dv1, s_v, w, thr)
    spk = slayer.spike.Spike.apply(vol, thr, tau, rho, graded, 0, 2)
    spk.backward(g)
    # fused
    x2, di2, dv2 = x.clone().requires_grad_(), d_i.clone().requires_grad_(), d_v.clone().requires_grad_()
    f_cur, f_vol, f_spk = D.cuba_fused.dynamics(x2, di2, dv2, s_i, s_v, w, thr, tau, rho, graded, 2)
    f_spk.backward(g)
    assert float(spk.detach().abs().sum()) > 0
    assert torch.equal(f_cur, cur.detach()), 'fused current differs'
    assert torch.equal(f_vol, vol.detach()), 'fused voltage differs'
    assert torch.equal(f_spk.detach(), spk.detach()), 'fused spikes differ'
    assert_same_gradient(x2.grad, x1.grad, 'fused grad_input differs')
    assert_rel(di2.grad.cpu(), di1.grad.cpu(), 'fused grad current_decay')
    assert_rel(dv2.grad.cpu(), dv1.grad.cpu(), 'fused grad voltage_decay')


def test_cuba_neuron_forward_uses_fused_path_with_same_results(slayer):
    gen = torch.Generator().manual_seed(104)
    x = sparse_input(gen, (3, 6, 5, 90), p=0.2).to(dev())
    torch.manual_seed(3)
    a = slayer.neuron.cuba.Neuron(1.0, [0.2, 0.4], [0.02, 0.2], shared_param=False, requires_grad=True,
                                  persistent_state=True).to(dev())
    b = slayer.neuron.cuba.Neuron(1.0, [0.2, 0.4], [0.02, 0.2], shared_param=False, requires_grad=True,
                                  persistent_state=True).to(dev())
    b._prepare(x)
    a._prepare(x)
    for pa, pb in zip(a.parameters(), b.parameters()):
        pb.data = pa.data.clone()
    for k in range(2):                                    # two calls: the carried state must agree too
        xa, xb = x.clone().requires_grad_(), x.clone().requires_grad_()
        sa = a(xa)                                        # fused
        _, vol = b.dynamics(xb)
        sb = b.spike(vol)                                 # three operators
        assert torch.equal(sa.detach(), sb.detach()), f'call {k}: spikes differ'
        assert torch.equal(a.voltage_state, b.voltage_state) and torch.equal(a.current_state, b.current_state)
        sa.sum().backward()
        sb.sum().backward()
        assert torch.equal(xa.grad, xb.grad)


@pytest.mark.parametrize('shape,w,graded', [((4, 128, 200), 64, False), ((3, 70, 129), 100, False),
                                            ((2, 3, 5, 7, 37), 4096, True), ((4, 9000, 64), 64, False),
                                            ((4, 70000, 40), 64, False)])
def test_fused_rf_equals_the_operator_chain(slayer, shape, w, graded):
    from tests.util import seed_of
    gen = torch.Generator().manual_seed(seed_of(shape, w, graded, 'rf fused'))
    C = shape[1]
    xr = sparse_input(gen, shape, p=0.2, amp=1.5).to(dev())
    xi = sparse_input(gen, shape, p=0.2, amp=1.5).to(dev())
    g = torch.randn(shape, generator=gen).to(dev())
    mag = torch.rand(C, generator=gen) * 4000
    ph = torch.rand(C, generator=gen) * 1.5
    sin, cos = (mag * torch.sin(ph)).round().to(dev()), (mag * torch.cos(ph)).round().to(dev())
    rs = torch.randn(shape[:-1], generator=gen).to(dev())
    is_ = torch.randn(shape[:-1], generator=gen).to(dev())
    last = torch.randn(shape[:-1], generator=gen).to(dev())
    thr, tau, rho = 0.6, 0.5, 10.0
    D = slayer.neuron.dynamics
    a = [t.clone().requires_grad_() for t in (xr, xi, sin, cos)]
    re, im = D.resonator.dynamics(a[0], a[1], a[2], a[3], rs, is_, w)
    spk = slayer.spike.complex.Spike.apply(re, im, thr, tau, rho, graded, last, 2)
    spk.backward(g)
    b = [t.clone().requires_grad_() for t in (xr, xi, sin, cos)]
    f_re, f_im, f_spk = D.rf_fused.dynamics(b[0], b[1], b[2], b[3], rs, is_, last, w, thr, tau, rho, graded, 2)
    f_spk.backward(g)
    assert float(spk.detach().abs().sum()) > 0
    assert torch.equal(f_re, re.detach()) and torch.equal(f_im, im.detach()), 'fused traces differ'
    assert torch.equal(f_spk.detach(), spk.detach()), 'fused spikes differ'
    assert_same_gradient(b[0].grad, a[0].grad, 'fused real input gradient differs')
    assert_same_gradient(b[1].grad, a[1].grad, 'fused imag input gradient differs')
    assert_rel(b[2].grad.cpu(), a[2].grad.cpu(), 'fused grad sin')
    assert_rel(b[3].grad.cpu(), a[3].grad.cpu(), 'fused grad cos')
    # without trainable decays the surrogate moves out of the sequential loop: same input gradients
    c = [xr.clone().requires_grad_(), xi.clone().requires_grad_()]
    l_spk = D.rf_fused.dynamics(c[0], c[1], sin, cos, rs, is_, last, w, thr, tau, rho, graded, 2)[2]
    l_spk.backward(g)
    assert_same_gradient(c[0].grad, a[0].grad, 'lean real input gradient differs')
    assert_same_gradient(c[1].grad, a[1].grad, 'lean imag input gradient differs')


@pytest.mark.parametrize('w', [64, 100, 4096, 3])
@pytest.mark.parametrize('graded', [False, True])
def test_fused_rf_spike_decision_on_integer_states(slayer, w, graded):
    """The fused forward decides the spike on the integer states.  No rotation (sin 0, cos 4096): the real part
    walks through every integer around threshold * w_scale while the imaginary part alternates in sign, for
    thresholds that are and are not multiples of 1 / w_scale, negative, zero, beyond the int range, NaN."""
    D = slayer.neuron.dynamics
    T = 64
    steps = torch.arange(T)
    for thr in (0.7, 1.0, 70 / w, (70 + 0.5) / w, -0.3, 0.0, 1e12, -1e12, float('nan')):
        centre = 0 if thr != thr or abs(thr) > 1e6 else int(round(thr * w))
        # row n: real state centre - 8 + n after step 0, then constant; imag -1, +1, -1, ... (units of 1 / w)
        xr = torch.zeros(16, 1, T)
        xr[:, 0, 0] = (centre - 8 + torch.arange(16)).float() / w
        xi = torch.zeros(16, 1, T)
        xi[:, 0, 0] = -1.0 / w
        xi[:, 0, 1:] = torch.where(steps[1:] % 2 == 1, 2.0, -2.0) / w      # +2, -2, +2, ...: the sign flips every step
        sin, cos = torch.tensor([0.0]), torch.tensor([4096.0])
        zero = torch.zeros(1)
        args = [t.to(dev()) for t in (xr, xi, sin, cos, zero, zero)]
        for last in (-1.0, 0.0, 1.0):
            lastt = torch.full((16, 1), last, device=dev())
            re, im = D.resonator.dynamics(*args, w)
            spk = slayer.spike.complex.Spike.apply(re, im, thr, 0.5, 10.0, graded, lastt, 2)
            f_re, f_im, f_spk = D.rf_fused.dynamics(*args, lastt, w, thr, 0.5, 10.0, graded, 2)
            assert torch.equal(f_re, re) and torch.equal(f_im, im)
            assert torch.equal(f_spk, spk), (w, thr, last, graded)
            _, _, i_spk = D.rf_fused.spikes(*args, lastt, w, thr, graded, 2)
            assert torch.equal(i_spk, spk), (w, thr, last, graded)
        if thr == thr and abs(thr) < 1e6:
            assert 0 < float((spk != 0).float().mean()) < 1, 'both outcomes must occur'


def test_rf_neuron_forward_uses_fused_path_with_same_results(slayer):
    gen = torch.Generator().manual_seed(105)
    shape = (3, 12, 150)
    xr, xi = sparse_input(gen, shape, p=0.3).to(dev()), sparse_input(gen, shape, p=0.3).to(dev())
    mk = lambda: slayer.neuron.rf.Neuron(1.0, [5, 20], [0.02, 0.1], shared_param=False, requires_grad=True,
                                         persistent_state=True).to(dev())
    a, b = mk(), mk()
    a._prepare(xr)
    b._prepare(xr)
    for pa, pb in zip(a.parameters(), b.parameters()):
        pb.data = pa.data.clone()
    for k in range(2):
        ia = (xr.clone().requires_grad_(), xi.clone().requires_grad_())
        ib = (xr.clone().requires_grad_(), xi.clone().requires_grad_())
        sa = a(ia)
        sb = b.spike(*b.dynamics(ib))
        assert torch.equal(sa.detach(), sb.detach()), f'call {k}: spikes differ'
        assert torch.equal(a.real_state, b.real_state) and torch.equal(a.imag_state, b.imag_state)
        sa.sum().backward()
        sb.sum().backward()
        assert torch.equal(ia[0].grad, ib[0].grad) and torch.equal(ia[1].grad, ib[1].grad)


@pytest.mark.parametrize('shape,w,graded', [((4, 128, 200), 64, False), ((3, 70, 129), 100, False),
                                            ((2, 3, 5, 7, 37), 4096, True), ((4, 9000, 64), 64, False),
                                            ((4, 70000, 40), 64, True)])
def test_fused_alif_equals_the_operator_chain(slayer, shape, w, graded):
    from tests.util import seed_of
    gen = torch.Generator().manual_seed(seed_of(shape, w, graded, 'alif fused'))
    C = shape[1]
    x = sparse_input(gen, shape, p=0.3, amp=2.0).to(dev())
    g = torch.randn(shape, generator=gen).to(dev())
    d_i, d_v, d_th, d_ref = (torch.randint(0, 4096, (C,), generator=gen).float().to(dev()) for _ in range(4))
    s_i, s_v = (torch.randn(shape[:-1], generator=gen).to(dev()) for _ in range(2))
    s_th = (1.0 + torch.rand(shape[:-1], generator=gen)).to(dev())
    s_ref = torch.rand(shape[:-1], generator=gen).to(dev())
    step, base, tau, rho = 0.5, 1.0, 0.7, 1.5
    D = slayer.neuron.dynamics
    a = [t.clone().requires_grad_() for t in (x, d_i, d_v)]
    cur = D.leaky_integrator.dynamics(a[0], a[1], s_i, w)
    vol = D.leaky_integrator.dynamics(cur, a[2], s_v, w)
    th, ref = D.adaptive_threshold.dynamics(vol, s_ref, d_ref, s_th, d_th, step, base, w)
    spk = slayer.spike.Spike.apply(vol, th + ref, tau, rho, graded, s_v, 2)
    spk.backward(g)
    b = [t.clone().requires_grad_() for t in (x, d_i, d_v)]
    f_cur, f_vol, f_theta, f_spk, f_th, f_ref = D.alif_fused.dynamics(
        b[0], b[1], b[2], d_th, d_ref, s_i, s_v, s_th, s_ref, step, base, w, tau, rho, graded, 2)
    f_spk.backward(g)
    assert 0 < float((spk.detach() != 0).float().mean()) < 1
    assert torch.equal(f_cur, cur.detach()) and torch.equal(f_vol, vol.detach()), 'fused traces differ'
    assert torch.equal(f_theta, (th + ref).detach()), 'fused threshold + refractory differs'
    assert torch.equal(f_th, th[..., -1]) and torch.equal(f_ref, ref[..., -1]), 'fused final states differ'
    assert torch.equal(f_spk.detach(), spk.detach()), 'fused spikes differ'
    assert_same_gradient(b[0].grad, a[0].grad, 'fused input gradient differs')
    assert_rel(b[1].grad.cpu(), a[1].grad.cpu(), 'fused grad current decay')
    assert_rel(b[2].grad.cpu(), a[2].grad.cpu(), 'fused grad voltage decay')


def test_alif_neuron_forward_uses_fused_path_with_same_results(slayer):
    gen = torch.Generator().manual_seed(106)
    shape = (3, 12, 150)
    x = sparse_input(gen, shape, p=0.3, amp=2.0).to(dev())
    mk = lambda: slayer.neuron.alif.Neuron(1.0, 0.5, [0.25, 0.3], [0.05, 0.1], [0.1, 0.2], [0.2, 0.3],
                                           shared_param=False, requires_grad=True, persistent_state=True).to(dev())
    a, b = mk(), mk()
    a._prepare(x)                                   # per-channel decays are drawn at random on the first call
    b._prepare(x)
    for pa, pb in zip(a.parameters(), b.parameters()):
        pb.data = pa.data.clone()
    for k in range(3):
        xa, xb = x.clone().requires_grad_(), x.clone().requires_grad_()
        sa = a(xa)
        _, vol, th, ref = b.dynamics(xb)
        sb = b.spike(vol, th, ref)
        assert torch.equal(sa.detach(), sb.detach()), f'call {k}: spikes differ'
        for name in ('current_state', 'voltage_state', 'threshold_state', 'refractory_state'):
            assert torch.equal(getattr(a, name), getattr(b, name)), f'call {k}: {name} differs'
        sa.sum().backward()
        sb.sum().backward()
        assert torch.equal(xa.grad, xb.grad), f'call {k}: input gradients differ'
    assert float(sa.detach().sum()) > 0


@pytest.mark.parametrize('shape,w', [((4, 128, 200), 64), ((3, 70, 129), 100), ((4, 9000, 64), 4096)])
def test_fused_cuba_without_current_trace(slayer, shape, w):
    """keep_current=False skips the current trace: same voltage, spikes and input gradient, and the
    last current comes back per neuron."""
    from tests.util import seed_of
    gen = torch.Generator().manual_seed(seed_of(shape, w, 'lean cuba'))
    C = shape[1]
    x = sparse_input(gen, shape, p=0.2, amp=1.5).to(dev())
    g = torch.randn(shape, generator=gen).to(dev())
    d_i, d_v = (torch.randint(0, 4096, (C,), generator=gen).float().to(dev()) for _ in range(2))
    s_i, s_v = (torch.randn(shape[:-1], generator=gen).to(dev()) for _ in range(2))
    F = slayer.neuron.dynamics.cuba_fused
    a, b = x.clone().requires_grad_(), x.clone().requires_grad_()
    cur, vol, spk = F.dynamics(a, d_i, d_v, s_i, s_v, w, 1.0, 0.7, 1.5)
    spk.backward(g)
    cur_last, vol2, spk2 = F.dynamics(b, d_i, d_v, s_i, s_v, w, 1.0, 0.7, 1.5, keep_current=False)
    spk2.backward(g)
    assert cur_last.shape == shape[:-1] and torch.equal(cur_last, cur[..., -1])
    assert torch.equal(vol2, vol) and torch.equal(spk2.detach(), spk.detach()) and float(spk.detach().sum()) > 0
    assert torch.equal(b.grad, a.grad)
    # trainable decays still get their gradients: the flag is ignored then
    dd = d_i.clone().requires_grad_()
    c3, _, s3 = F.dynamics(x, dd, d_v, s_i, s_v, w, 1.0, 0.7, 1.5, keep_current=False)
    s3.backward(g)
    assert c3.shape == shape and dd.grad is not None and torch.isfinite(dd.grad).all()


@pytest.mark.parametrize('shape,w', [((4, 128, 200), 64), ((3, 70, 129), 100)])
def test_fused_alif_without_current_trace(slayer, shape, w):
    from tests.util import seed_of
    gen = torch.Generator().manual_seed(seed_of(shape, w, 'lean alif'))
    C = shape[1]
    x = sparse_input(gen, shape, p=0.3, amp=2.0).to(dev())
    g = torch.randn(shape, generator=gen).to(dev())
    decays = [torch.randint(0, 4096, (C,), generator=gen).float().to(dev()) for _ in range(4)]
    states = [torch.rand(shape[:-1], generator=gen).to(dev()) for _ in range(4)]
    states[2] = states[2] + 1.0
    F = slayer.neuron.dynamics.alif_fused
    a, b = x.clone().requires_grad_(), x.clone().requires_grad_()
    full = F.dynamics(a, *decays, *states, 0.5, 1.0, w, 0.7, 1.5)
    full[3].backward(g)
    lean = F.dynamics(b, *decays, *states, 0.5, 1.0, w, 0.7, 1.5, keep_current=False)
    lean[3].backward(g)
    assert lean[0].shape == shape[:-1] and torch.equal(lean[0], full[0][..., -1])
    for i in (1, 2, 4, 5):
        assert torch.equal(lean[i], full[i]), f'output {i} differs'
    assert torch.equal(lean[3].detach(), full[3].detach()) and float(full[3].detach().sum()) > 0
    assert torch.equal(b.grad, a.grad)


@pytest.mark.parametrize('kind', ['cuba', 'alif', 'rf'])
@pytest.mark.parametrize('shared', [True, False])
def test_neuron_inference_form_matches_training_form(slayer, kind, shared):
    """Under no_grad only the spikes are written; spikes and the carried states must equal the
    training form over several calls with persistent state."""
    gen = torch.Generator().manual_seed(107)
    shape = (3, 12, 6, 152)
    rng = lambda a, b: [a, b] if not shared else a
    if kind == 'cuba':
        mk = lambda: slayer.neuron.cuba.Neuron(1.0, rng(0.2, 0.4), rng(0.02, 0.2), shared_param=shared,
                                               persistent_state=True).to(dev())
    elif kind == 'alif':
        mk = lambda: slayer.neuron.alif.Neuron(1.0, 0.5, rng(0.25, 0.4), rng(0.03, 0.2), rng(0.1, 0.3), rng(0.1, 0.3),
                                               shared_param=shared, persistent_state=True).to(dev())
    else:
        mk = lambda: slayer.neuron.rf.Neuron(1.0, rng(5, 20) if not shared else 11, rng(0.02, 0.1),
                                             shared_param=shared, persistent_state=True).to(dev())
    x = sparse_input(gen, shape, p=0.3, amp=2.0).to(dev())
    x2 = sparse_input(gen, shape, p=0.3, amp=2.0).to(dev())
    inp = (lambda grad: (x.clone().requires_grad_(grad), x2.clone().requires_grad_(grad))) if kind == 'rf' \
        else (lambda grad: x.clone().requires_grad_(grad))
    a, b = mk(), mk()
    a._prepare(x); b._prepare(x)
    for pa, pb in zip(a.parameters(), b.parameters()):
        pb.data = pa.data.clone()
    states = [n for n, _ in a.named_buffers() if n.endswith('_state')]
    total = 0.0
    for k in range(3):
        sa = a(inp(True))
        with torch.no_grad():
            sb = b(inp(False))
        assert torch.equal(sa.detach(), sb), f'call {k}: spikes differ'
        for name in states:
            assert torch.equal(getattr(a, name), getattr(b, name)), f'call {k}: {name} differs'
        total += float(sb.sum())
    assert total > 0 and len(states) >= 2


def test_fused_cuba_under_graph_capture_replays(slayer):
    """The entry points enqueue kernels only (no memset nodes, no allocation of their own), so a step
    can be captured in a graph; every replay, with eager work in between, must equal the eager result."""
    gen = torch.Generator().manual_seed(108)
    shape = (4, 16, 8, 96)
    F = slayer.neuron.dynamics.cuba_fused
    d_i, d_v = (torch.randint(0, 4096, (16,), generator=gen).float().to(dev()) for _ in range(2))
    zero = torch.zeros(1, device=dev())
    x = sparse_input(gen, shape, p=0.2, amp=1.5).to(dev())
    g = torch.randn(shape, generator=gen).to(dev())

    def step():
        cur, vol, spk = F._fwd(x, d_i, d_v, zero, zero, 64, 1.0, False, 1)
        g_x, g_i, g_v = F._bwd(g, vol, cur, d_i, d_v, 1.0, 1.0, 1.0, False)
        return spk, g_x, g_i, g_v

    step()                                      # warm-up outside the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        step()
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            outs = step()
    torch.cuda.synchronize()
    for k in range(4):
        x.copy_(sparse_input(gen, shape, p=0.2, amp=1.5).to(dev()))
        g.copy_(torch.randn(shape, generator=gen).to(dev()))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outs]
        want = step()                           # eager work between the replays
        torch.cuda.synchronize()
        assert float(want[0].sum()) > 0
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a, b), f'replay {k}: output {i} differs from the eager result'


@pytest.mark.parametrize('w', [4096, 1000])
def test_fused_blocks_equal_the_chains_beyond_float32_integers(slayer, w):
    from tests.util import seed_of
    """Barely any decay and a biased input: the integer states pass 2**24, where the int -> float32 conversion at
    every operator boundary rounds.  The fused CUBA / ALIF / RF blocks make the same round trips, so traces,
    spikes and final states still equal the operator chains bit for bit (full, lean and inference forms)."""
    gen = torch.Generator().manual_seed(seed_of('beyond 2**24', w))
    D = slayer.neuron.dynamics
    shape = (2, 24, 800)
    C = shape[1]
    x = (0.2 + 0.3 * torch.rand(shape, generator=gen)).to(dev())
    zero = torch.zeros(1, device=dev())
    d_i = torch.randint(0, 3, (C,), generator=gen).float().to(dev())
    d_v = torch.randint(0, 3, (C,), generator=gen).float().to(dev())
    # CUBA: threshold far up, so the voltage resets from states beyond 2**24
    thr = 2.0e4
    cur = D.leaky_integrator.dynamics(x, d_i, zero, w)
    vol = D.leaky_integrator.dynamics(cur, d_v, zero, w, thr)
    spk = slayer.spike.Spike.apply(vol, thr, 1.0, 1.0, False, 0, 1)
    assert float(vol.abs().max()) * w > 2 ** 24 and 0 < float(spk.sum()) < spk.numel() / 2
    f_cur, f_vol, f_spk = D.cuba_fused.dynamics(x, d_i, d_v, zero, zero, w, thr, 1.0, 1.0, False, 1)
    assert torch.equal(f_cur, cur) and torch.equal(f_vol, vol) and torch.equal(f_spk, spk), 'CUBA'
    l_cur, l_vol, l_spk = D.cuba_fused.dynamics(x, d_i, d_v, zero, zero, w, thr, 1.0, 1.0, False, 1, keep_current=False)
    assert torch.equal(l_cur, cur[..., -1]) and torch.equal(l_vol, vol) and torch.equal(l_spk, spk), 'CUBA lean'
    i_cur, i_vol, i_spk = D.cuba_fused.spikes(x, d_i, d_v, zero, zero, w, thr, False, 1)
    assert torch.equal(i_cur, cur[..., -1]) and torch.equal(i_vol, vol[..., -1]) and torch.equal(i_spk, spk), 'CUBA inference'
    # ALIF: no reset at all, the voltage keeps growing; threshold and refractory follow it
    d_th = torch.randint(0, 50, (C,), generator=gen).float().to(dev())
    d_ref = torch.randint(0, 50, (C,), generator=gen).float().to(dev())
    one = torch.ones(1, device=dev())
    # (a quarter of the drive: threshold and refractory state pass 2**24 but stay below 2**28, the bound beyond
    # which the kernels no longer vouch for 32 bits and raise their range flag)
    step, base = 3.0e3, 1.0e3
    xa = 0.25 * x
    cur_a = D.leaky_integrator.dynamics(xa, d_i, zero, w)
    vol2 = D.leaky_integrator.dynamics(cur_a, d_v, zero, w)
    th, ref = D.adaptive_threshold.dynamics(vol2, zero, d_ref, one * base, d_th, step, base, w)
    spk2 = slayer.spike.Spike.apply(vol2, th + ref, 1.0, 1.0, False, 0, 1)
    assert float(vol2.abs().max()) * w > 2 ** 24 and float((th + ref).abs().max()) * w > 2 ** 24
    assert float(th.abs().max()) * w < 2 ** 28 and float(ref.abs().max()) * w < 2 ** 28
    assert 0 < float(spk2.sum()) < spk2.numel()
    f = D.alif_fused.dynamics(xa, d_i, d_v, d_th, d_ref, zero, zero, one * base, zero, step, base, w, 1.0, 1.0, False, 1)
    assert torch.equal(f[0], cur_a) and torch.equal(f[1], vol2) and torch.equal(f[2], th + ref), 'ALIF traces'
    assert torch.equal(f[3], spk2) and torch.equal(f[4], th[..., -1]) and torch.equal(f[5], ref[..., -1]), 'ALIF'
    s = D.alif_fused.spikes(xa, d_i, d_v, d_th, d_ref, zero, zero, one * base, zero, step, base, w, False, 1)
    assert torch.equal(s[3], spk2) and torch.equal(s[4], th[..., -1]) and torch.equal(s[5], ref[..., -1]), 'ALIF inference'
    # RF: slow rotation with a gain just below one, biased input on both parts
    ph = torch.linspace(0.002, 0.02, C)
    sin, cos = (4095 * torch.sin(ph)).round().to(dev()), (4095 * torch.cos(ph)).round().to(dev())
    x = 100 * x
    square = torch.where(torch.arange(shape[-1]) % 100 < 50, 1.0, -1.0)       # the imaginary part swings through zero
    xi = (1500 * torch.rand(shape, generator=gen) * square).to(dev())
    re, im = D.resonator.dynamics(x, xi, sin, cos, zero, zero, w)
    thr_rf = 5.0e3
    spk3 = slayer.spike.complex.Spike.apply(re, im, thr_rf, 0.5, 10.0, False, 0, 1)
    assert float(re.abs().max()) * w > 2 ** 24 and 0 < float(spk3.sum()) < spk3.numel()
    f_re, f_im, f_spk3 = D.rf_fused.dynamics(x, xi, sin, cos, zero, zero, zero, w, thr_rf, 0.5, 10.0, False, 1)
    assert torch.equal(f_re, re) and torch.equal(f_im, im) and torch.equal(f_spk3, spk3), 'RF'
    r_last, i_last, i_spk3 = D.rf_fused.spikes(x, xi, sin, cos, zero, zero, zero, w, thr_rf, False, 1)
    assert torch.equal(r_last, re[..., -1]) and torch.equal(i_last, im[..., -1]) and torch.equal(i_spk3, spk3), 'RF inference'


def test_cuba_neuron_with_a_norm_takes_the_operator_chain(slayer):
    """A normalisation sits between current and voltage, so the fused block cannot be used: forward must be
    current -> norm (with the neuron's quantiser hooked in) -> voltage with reset -> spike."""
    gen = torch.Generator().manual_seed(310)
    x = sparse_input(gen, (4, 10, 120), p=0.3, amp=2.0).to(dev())
    n = slayer.neuron.cuba.Neuron(1.0, 0.25, 0.05, norm=slayer.neuron.norm.MeanOnlyBatchNorm).to(dev())
    n.eval()
    n.norm.running_mean = (torch.rand(10, generator=gen) * 0.4).to(dev())
    spk = n(x)
    D = slayer.neuron.dynamics
    zero = torch.zeros(1, device=dev())
    cur = D.leaky_integrator.dynamics(x, torch.tensor([1024.0], device=dev()), zero, 4096)
    shift = n.quantize_8bit(n.norm.running_mean).reshape(1, -1, 1)
    assert float(shift.abs().max()) > 0 and torch.equal(shift * 32, torch.round(shift * 32))     # steps of 2 / 64
    vol = D.leaky_integrator.dynamics(cur - shift, torch.tensor([205.0], device=dev()), zero, 4096, 1.0 + 0.01 / 4096)
    want = slayer.spike.Spike.apply(vol, 1.0 + 0.01 / 4096, 100.0, 0.1, False, 0, 1)
    assert 0 < float(want.sum()) < want.numel()
    assert torch.equal(spk, want)
    assert torch.equal(n.norm.bias, -n.quantize_8bit(n.norm.running_mean, descale=True))


@pytest.mark.parametrize('kind', ['cuba', 'alif'])
@pytest.mark.parametrize('trained', [False, True])
def test_fused_neurons_round_their_decays_like_the_quantizer(slayer, kind, trained):
    """Decays that are not integers, halves among them (round-half-even): the fused kernels take the parameters
    as they are and round them themselves; the operator chain gets quantize(decay) from the neuron class."""
    gen = torch.Generator().manual_seed(991)
    x = sparse_input(gen, (3, 4, 7, 120), p=0.3, amp=1.5).to(dev())
    decays = [[1000.5, 1001.5, 409.6, 37.49], [300.5, 12.5, 2047.51, 0.4]]
    if kind == 'cuba':
        mk = lambda: slayer.neuron.cuba.Neuron(1.0, [0.2, 0.4], [0.1, 0.3], shared_param=False, requires_grad=trained,
                                               persistent_state=True).to(dev())
    else:
        mk = lambda: slayer.neuron.alif.Neuron(1.0, 0.5, [0.2, 0.4], [0.1, 0.3], [0.1, 0.3], [0.2, 0.4],
                                               shared_param=False, requires_grad=trained,
                                               persistent_state=True).to(dev())
    a, b = mk(), mk()
    a._prepare(x)
    b._prepare(x)
    for n in (a, b):
        with torch.no_grad():
            n.current_decay.copy_(torch.tensor(decays[0]))
            n.voltage_decay.copy_(torch.tensor(decays[1]))
            if kind == 'alif':
                n.threshold_decay.copy_(torch.tensor([100.5, 101.5, 77.7, 3.2]))
                n.refractory_decay.copy_(torch.tensor([600.5, 601.5, 15.5, 900.49]))
    for grad in (False, True):
        xa, xb = x.clone().requires_grad_(grad), x.clone().requires_grad_(grad)
        with torch.set_grad_enabled(grad):
            sa = a(xa)                                                   # fused
            sb = b.spike(*b.dynamics(xb)[1:])                            # separate operators
        assert float(sa.detach().sum()) > 0
        assert torch.equal(sa.detach(), sb.detach()), f'spikes differ (grad={grad})'
        assert torch.equal(a.voltage_state, b.voltage_state) and torch.equal(a.current_state, b.current_state)
        if grad:
            sa.sum().backward()
            sb.sum().backward()
            assert_same_gradient(xa.grad, xb.grad, 'input gradient')
