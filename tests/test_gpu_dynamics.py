"""GPU parity of the fixed-point dynamics kernels against the CPU oracle, through the
python operator interface (ctypes -> C ABI -> HIP kernels).  Integer-mode outputs must
be bit-exact; float-mode gradients within 1e-5 relative."""
import numpy as np
import pytest
import torch

from oracle import slayer_oracle as O
from tests.golden import fixtures as G
from tests.util import (assert_exact, assert_rel, assert_same_gradient, assert_scale, assert_sum, dev, li_decay_grad_f64,
                        res_decay_grads_f64, seed_of, sparse_input, SCAN_MIN)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope='module')
def slayer():
    import lava_dl_amd.slayer as s
    return s


def _decay(kind, shape, gen):
    C = shape[1]
    spatial = shape[1:-1]
    if kind == 'shared':
        return torch.tensor([float(torch.randint(0, 4097, (1,), generator=gen))])
    if kind == 'channel':
        return torch.randint(0, 4097, (C,), generator=gen).float()
    return torch.randint(0, 4097, tuple(spatial), generator=gen).float()


LI_CASES = [
    # shape,               decay kind, w,    threshold,          state
    ((4, 128, 200),        'shared',   64,   1.25,               'scalar'),
    ((4, 128, 200),        'channel',  64,   None,               'full'),
    ((2, 16, 8, 8, 300),   'channel',  64,   1.0,                'scalar'),
    ((2, 3, 5, 7, 37),     'channel',  4096, 1.0 + 0.01 / 4096,  'full'),     # T % 4 != 0, M % 64 != 0
    ((3, 70, 129),         'neuron',   100,  0.77,               'full'),     # w not a power of two
    ((1, 5, 3),            'neuron',   64,   None,               'scalar'),   # T < 4
    ((2, 64, 1),           'channel',  64,   0.5,                'full'),     # T == 1
    ((1, 1, 260),          'shared',   4096, 2.0,                'scalar'),   # one neuron
    ((2, 130, 64),         'channel',  64,   0.0,                'scalar'),   # threshold 0 = disabled
    ((3, 50, 36),          'channel',  64,   1.0,                'scalar'),   # rows barely longer than a 128-byte line
    ((3, 50, 28),          'channel',  64,   1.0,                'full'),     # rows shorter than a line
    ((1, 67, 300),         'channel',  64,   1.0,                'scalar'),   # partial last wave, T % 32 == 12
    ((2, 64, 100),         'neuron',   64,   1.0,                'scalar'),   # exactly one wave per batch element
    ((5, 33, 1000),        'channel',  4096, 1.0,                'full'),     # T % 32 == 8
]


@pytest.mark.parametrize('shape,kind,w,thr,state_kind', LI_CASES)
def test_li_fwd_bit_exact(slayer, shape, kind, w, thr, state_kind):
    gen = torch.Generator().manual_seed(seed_of(shape, kind, w))
    x = sparse_input(gen, shape, p=0.1, amp=2.0)
    decay = _decay(kind, shape, gen)
    state = torch.tensor([0.0]) if state_kind == 'scalar' else torch.randn(shape[:-1], generator=gen)
    ref = O.li_fwd(x, decay, state, w, thr)
    out = slayer.neuron.dynamics.leaky_integrator.dynamics(
        x.to(dev()), decay.to(dev()), state.to(dev()), w, thr)
    assert_exact(out, ref, f'li_fwd {shape}')


@pytest.mark.parametrize('M_per_batch', [70000, 35000, 9000, 2000])
def test_all_tile_geometries(slayer, M_per_batch):
    """Each kernel picks 64, 32 or 16 rows per wave from the neuron count (thresholds at 262144, 65536 and
    16384 neurons depending on the kernel); every geometry must give the same bits.  The four sizes
    here (280000, 140000, 36000, 8000 neurons) reach every instantiation."""
    N, T = 4, 100
    shape = (N, M_per_batch, T)
    gen = torch.Generator().manual_seed(seed_of(shape))
    x = sparse_input(gen, shape, p=0.1, amp=2.0)
    d1 = torch.randint(0, 4097, (M_per_batch,), generator=gen).float()
    d2 = torch.randint(0, 4097, (M_per_batch,), generator=gen).float()
    zero, one = torch.tensor([0.0]), torch.tensor([1.0])
    xg, d1g, d2g, zg, og = x.to(dev()), d1.to(dev()), d2.to(dev()), zero.to(dev()), one.to(dev())
    D = slayer.neuron.dynamics
    ref = O.li_fwd(x, d1, zero, 64, 1.0)
    out = D.leaky_integrator.dynamics(xg, d1g, zg, 64, 1.0)
    assert_exact(out, ref, 'li_fwd')
    g = torch.randn(shape, generator=gen)
    from lava_dl_amd.slayer.neuron.dynamics import leaky_integrator as L, resonator as R
    gi, gd = L._bwd(g.to(dev()), out, d1g)
    r_gi, r_gd = O.li_bwd(g, ref, d1)
    (assert_exact if gi.numel() < SCAN_MIN else assert_scale)(gi, r_gi, 'li_bwd grad_input')
    assert_sum(gd, *li_decay_grad_f64(gi, out, M_per_batch), 'li_bwd grad_decay')
    th, rf = D.adaptive_threshold.dynamics(xg, zg, d1g, og, d2g, 0.5, 1.0, 64)
    r_th, r_rf = O.ath_fwd(x, zero, d1, one, d2, 0.5, 1.0, 64)
    assert_exact(th, r_th, 'ath threshold')
    assert_exact(rf, r_rf, 'ath refractory')
    x2 = sparse_input(gen, shape, p=0.1, amp=2.0)
    sin, cos = (d1 * 0.6).round(), (d2 * 0.7).round()
    re, im = D.resonator.dynamics(xg, x2.to(dev()), sin.to(dev()), cos.to(dev()), zg, zg, 64)
    r_re, r_im = O.res_fwd(x, x2, sin, cos, zero, zero, 64)
    assert_exact(re, r_re, 'res real')
    assert_exact(im, r_im, 'res imag')
    got = R._bwd(g.to(dev()), xg, re, im, sin.to(dev()), cos.to(dev()))
    want = O.res_bwd(g, x, r_re, r_im, sin, cos)
    close = assert_exact if got[0].numel() < SCAN_MIN else assert_scale
    close(got[0], want[0], 'res_bwd grad_real')
    close(got[1], want[1], 'res_bwd grad_imag')
    s_sum, s_mag, c_sum, c_mag = res_decay_grads_f64(got[0], got[1], re, im, M_per_batch)
    assert_sum(got[2], s_sum, s_mag, 'res_bwd grad_sin')
    assert_sum(got[3], c_sum, c_mag, 'res_bwd grad_cos')


@pytest.mark.parametrize('thr', [4100.0, 4096.0 + 1.0 / 4096, 7000.3, 16384.0])
def test_li_fwd_reset_decision_on_states_beyond_float32_integers(slayer, thr):
    """The kernel decides the reset on the integer state; the reference compares float32(state) with
    float32(threshold * w).  Beyond 2**24 the conversion rounds, so states next to such a threshold
    check that both decisions agree."""
    gen = torch.Generator().manual_seed(seed_of('big states', thr))
    shape, w = (2, 64, 400), 4096
    # no decay; now and then a jump to just below threshold * w >= 2**24, then steps of a few LSB
    jump = (torch.rand(shape, generator=gen) < 0.1).float()
    x = jump * (thr - torch.randint(0, 6, shape, generator=gen).float() / w) \
        + (1 - jump) * torch.randint(-2, 4, shape, generator=gen).float() / w
    decay = torch.tensor([0.0])
    state = torch.tensor([0.0])
    ref = O.li_fwd(x, decay, state, w, thr)
    fired = (ref * w >= thr * w).float().mean()
    assert 0.02 < float(fired) < 0.5, 'the case must cross the threshold both ways'
    out = slayer.neuron.dynamics.leaky_integrator.dynamics(x.to(dev()), decay.to(dev()), state.to(dev()), w, thr)
    assert_exact(out, ref, f'li_fwd big states thr={thr}')


def test_big_state_vectors_of_the_reference_cpu_branch(slayer):
    """Vectors computed by the reference itself (tests/golden/make_reference_vectors.py): leaky integrator and
    thresholded resonator with states beyond 2**24, vector kernels and one-thread-per-neuron kernels."""
    li, res = G.reference_big_state_vectors()
    D = slayer.neuron.dynamics
    zero = torch.tensor([0.0], device=dev())
    for case in li:
        for debug in (False, True):
            out = D.leaky_integrator.dynamics(case['x'].to(dev()), zero, zero, G.W_SCALE, case['threshold'], debug=debug)
            assert_exact(out, case['out'], f"li reference vectors thr={case['threshold']} debug={debug}")
    for case in res:
        for debug in (False, True):
            re, im = D.resonator.dynamics(case['xr'].to(dev()), case['xi'].to(dev()), case['sin'].to(dev()),
                                          case['cos'].to(dev()), zero, zero, G.W_SCALE, case['threshold'], debug=debug)
            assert_exact(re, case['re'], f"res reference vectors real thr={case['threshold']} debug={debug}")
            assert_exact(im, case['im'], f"res reference vectors imag thr={case['threshold']} debug={debug}")


def test_li_fwd_negative_and_edge_decays(slayer):
    gen = torch.Generator().manual_seed(7)
    x = sparse_input(gen, (2, 8, 96), p=0.5, amp=30.0)
    decay = torch.tensor([0.0, 1.0, 2047.0, 4095.0, 4096.0, 1234.7, 5000.0, -17.0])
    state = torch.randn(2, 8, generator=gen) * 50
    for thr in (None, 3.0):
        ref = O.li_fwd(x, decay, state, 64, thr)
        out = slayer.neuron.dynamics.leaky_integrator.dynamics(x.to(dev()), decay.to(dev()), state.to(dev()), 64, thr)
        assert_exact(out, ref, f'li_fwd edge decays thr={thr}')


def test_li_fwd_non_contiguous_and_offset_views(slayer):
    gen = torch.Generator().manual_seed(8)
    base = sparse_input(gen, (3, 40, 101), p=0.2)
    decay = torch.tensor([300.0])
    zero = torch.tensor([0.0])
    xg = base.to(dev())
    # a view that starts 4 bytes into the allocation and has T % 4 != 0
    v_cpu, v_gpu = base[:, :, 1:], xg[:, :, 1:]
    assert_exact(slayer.neuron.dynamics.leaky_integrator.dynamics(v_gpu, decay.to(dev()), zero.to(dev()), 64, 1.0),
                 O.li_fwd(v_cpu.contiguous(), decay, zero, 64, 1.0), 'li_fwd strided view')
    # contiguous but misaligned base pointer with T % 4 == 0
    flat = torch.zeros(2 * 64 * 100 + 1)
    flat[1:] = sparse_input(gen, (2 * 64 * 100,), p=0.2)
    fg = flat.to(dev())
    v_cpu, v_gpu = flat[1:].reshape(2, 64, 100), fg[1:].reshape(2, 64, 100)
    assert v_gpu.data_ptr() % 16 != 0
    assert_exact(slayer.neuron.dynamics.leaky_integrator.dynamics(v_gpu, decay.to(dev()), zero.to(dev()), 64, 1.0),
                 O.li_fwd(v_cpu, decay, zero, 64, 1.0), 'li_fwd misaligned base')


def test_li_empty(slayer):
    z = torch.zeros(0, 4, 10, device=dev())
    out = slayer.neuron.dynamics.leaky_integrator.dynamics(z, torch.tensor([1.0], device=dev()),
                                                           torch.tensor([0.0], device=dev()), 64)
    assert out.shape == z.shape


def test_li_rejects_cpu_and_wrong_dtype(slayer):
    d = torch.tensor([1.0])
    with pytest.raises(RuntimeError):
        slayer.neuron.dynamics.leaky_integrator.dynamics(torch.zeros(1, 2, 8), d, d, 64)
    with pytest.raises(RuntimeError):
        slayer.neuron.dynamics.leaky_integrator.dynamics(torch.zeros(1, 2, 8, device=dev(), dtype=torch.float64),
                                                         d.to(dev()), d.to(dev()), 64)
    with pytest.raises(RuntimeError):   # 3 decays cannot map onto 4 channels
        slayer.neuron.dynamics.leaky_integrator.dynamics(torch.zeros(1, 4, 8, device=dev()),
                                                         torch.zeros(3, device=dev()), d.to(dev()), 64)


def test_dense_lif_fixture_on_gpu(slayer):
    """Reference-held known answer (netx gts/dense): CUBA current -> voltage -> spike."""
    fx = G.dense_lif()
    li = slayer.neuron.dynamics.leaky_integrator.dynamics
    zero = torch.tensor([0.0], device=dev())
    cur = li(fx['x'].to(dev()), torch.tensor([fx['current_decay']], device=dev()), zero, G.W_SCALE)
    vol = li(cur, torch.tensor([fx['voltage_decay']], device=dev()), zero, G.W_SCALE, fx['threshold'])
    spk = slayer.spike.Spike.apply(vol, fx['threshold'], 1.0, 1.0, False, 0, 1)
    got = spk[0].cpu().numpy().astype(np.int64)[:, :fx['expected'].shape[1]]
    assert int((got != fx['expected']).sum()) == 0
    assert got.sum() == 1826


@pytest.mark.parametrize('shape,kind', [((4, 128, 200), 'shared'), ((2, 16, 8, 8, 300), 'channel'),
                                        ((3, 70, 129), 'channel'), ((2, 3, 5, 7, 37), 'neuron'),
                                        ((2, 64, 1), 'channel'), ((1, 5, 3), 'shared')])
def test_li_bwd(slayer, shape, kind):
    gen = torch.Generator().manual_seed(seed_of(shape, kind))
    go = torch.randn(shape, generator=gen)
    out = torch.randn(shape, generator=gen)
    decay = _decay(kind, shape, gen)
    if kind == 'neuron':      # the reference reduces per-neuron decay gradients to [C]; not supported there either
        ref_g, _ = O.li_bwd(go, out, decay)
        ref_gd = (ref_g[..., 1:].double() * out[..., :-1].double()).sum(dim=(0, -1)).float()
    else:
        ref_g, ref_gd = O.li_bwd(go, out, decay)
    from lava_dl_amd.slayer.neuron.dynamics import leaky_integrator as L
    g, gd = L._bwd(go.to(dev()), out.to(dev()), decay.to(dev()))
    assert_exact(g, ref_g, f'li_bwd grad_input {shape}')      # same op order, no contraction -> identical bits
    assert_sum(gd, *li_decay_grad_f64(g, out, decay.numel()), f'li_bwd grad_decay {shape}')


def test_li_autograd_matches_oracle(slayer):
    gen = torch.Generator().manual_seed(11)
    x = sparse_input(gen, (2, 6, 4, 4, 60), p=0.1)
    decay = torch.randint(0, 4096, (6,), generator=gen).float()
    xg = x.to(dev()).requires_grad_()
    dg = decay.to(dev()).requires_grad_()
    out = slayer.neuron.dynamics.leaky_integrator.dynamics(xg, dg, torch.tensor([0.0], device=dev()), 64, 1.0)
    go = torch.randn(x.shape, generator=gen)
    out.backward(go.to(dev()))
    ref_out = O.li_fwd(x, decay, torch.tensor([0.0]), 64, 1.0)
    ref_g, ref_gd = O.li_bwd(go, ref_out, decay)
    assert_exact(out, ref_out, 'autograd fwd')
    assert_exact(xg.grad, ref_g, 'autograd grad_input')
    assert dg.grad.shape == decay.shape
    assert_rel(dg.grad, ref_gd, 'autograd grad_decay')


# ------------------------------------------------------------------------------------- ATH
ATH_CASES = [((4, 128, 200), 'channel', 64), ((2, 3, 5, 7, 37), 'channel', 4096), ((3, 70, 129), 'neuron', 100),
             ((2, 64, 1), 'shared', 64), ((1, 5, 3), 'shared', 64)]


@pytest.mark.parametrize('shape,kind,w', ATH_CASES)
def test_ath_fwd_bit_exact(slayer, shape, kind, w):
    gen = torch.Generator().manual_seed(seed_of(shape, kind, w, 'ath'))
    x = sparse_input(gen, shape, p=0.3, amp=3.0)
    rd, td = _decay(kind, shape, gen), _decay(kind, shape, gen)
    th_state = torch.rand(shape[:-1], generator=gen) * 2        # includes th < th0
    ref_state = torch.randn(shape[:-1], generator=gen)          # includes r < 0
    ref_th, ref_r = O.ath_fwd(x, ref_state, rd, th_state, td, 0.5, 1.0, w)
    th, r = slayer.neuron.dynamics.adaptive_threshold.dynamics(
        x.to(dev()), ref_state.to(dev()), rd.to(dev()), th_state.to(dev()), td.to(dev()), 0.5, 1.0, w)
    assert_exact(th, ref_th, f'ath threshold {shape}')
    assert_exact(r, ref_r, f'ath refractory {shape}')


def test_ath_scalar_states_and_no_grad(slayer):
    gen = torch.Generator().manual_seed(21)
    x = sparse_input(gen, (2, 32, 100), p=0.3, amp=3.0)
    one, zero = torch.tensor([1.0]), torch.tensor([0.0])
    rd, td = torch.tensor([300.0]), torch.tensor([100.0])
    ref_th, ref_r = O.ath_fwd(x, zero, rd, one, td, 0.5, 1.0, 64)
    xg = x.to(dev()).requires_grad_()
    th, r = slayer.neuron.dynamics.adaptive_threshold.dynamics(
        xg, zero.to(dev()), rd.to(dev()), one.to(dev()), td.to(dev()), 0.5, 1.0, 64)
    assert_exact(th, ref_th, 'ath th')
    assert_exact(r, ref_r, 'ath ref')
    (th.sum() + r.sum() + (xg * 2).sum()).backward()
    assert torch.equal(xg.grad.cpu(), torch.full(x.shape, 2.0))   # nothing flows back through the op


# ------------------------------------------------------------------------------------- RES
RES_CASES = [((4, 128, 200), 'channel', 64, None), ((2, 3, 5, 7, 37), 'channel', 4096, None),
             ((3, 70, 129), 'neuron', 100, 1.5), ((2, 64, 1), 'shared', 64, 0.0), ((1, 5, 3), 'shared', 64, 2.3),
             ((2, 40, 64), 'channel', 64, 1.0)]


def _rot(kind, shape, gen):
    n = _decay(kind, shape, gen).numel()
    vshape = _decay(kind, shape, gen).shape
    mag = torch.rand(n, generator=gen) * 4095
    ph = torch.rand(n, generator=gen) * 2 * np.pi
    return (mag * torch.sin(ph)).round().reshape(vshape), (mag * torch.cos(ph)).round().reshape(vshape)


@pytest.mark.parametrize('shape,kind,w,thr', RES_CASES)
def test_res_fwd_bit_exact(slayer, shape, kind, w, thr):
    gen = torch.Generator().manual_seed(seed_of(shape, kind, w, 'res'))
    xr = sparse_input(gen, shape, p=0.2, amp=2.0)
    xi = sparse_input(gen, shape, p=0.2, amp=2.0)
    sin, cos = _rot(kind, shape, gen)
    rs = torch.randn(shape[:-1], generator=gen)
    is_ = torch.randn(shape[:-1], generator=gen)
    ref_re, ref_im = O.res_fwd(xr, xi, sin, cos, rs, is_, w, thr)
    re, im = slayer.neuron.dynamics.resonator.dynamics(
        xr.to(dev()), xi.to(dev()), sin.to(dev()), cos.to(dev()), rs.to(dev()), is_.to(dev()), w, thr)
    assert_exact(re, ref_re, f'res real {shape}')
    assert_exact(im, ref_im, f'res imag {shape}')


def test_rf_fixtures_on_gpu(slayer):
    """Reference-held known answers (netx gts/complex_dense): RF dense block (phase spike, no
    reset) and RF_IZ input block (threshold mode with reset)."""
    res = slayer.neuron.dynamics.resonator.dynamics
    zero = torch.tensor([0.0], device=dev())
    fx = G.complex_dense_rf()
    re, im = res(fx['xr'].to(dev()), fx['xi'].to(dev()), torch.tensor([fx['sin_decay']], device=dev()),
                 torch.tensor([fx['cos_decay']], device=dev()), zero, zero, G.W_SCALE)
    spk = slayer.spike.complex.Spike.apply(re, im, fx['threshold'], 0.5, 10.0, False, 0, 1)
    got = spk[0].cpu().numpy().astype(np.int64)[:, :fx['expected'].shape[1]]
    assert int((got != fx['expected']).sum()) == 0 and got.sum() > 40000
    fx = G.complex_input_rf_iz()
    x = fx['x'].to(dev())
    re, im = res(x, x, torch.tensor([fx['sin_decay']], device=dev()), torch.tensor([fx['cos_decay']], device=dev()),
                 zero, zero, G.W_SCALE, fx['threshold'])
    got = (im >= fx['threshold'])[0].cpu().numpy().astype(np.int64)
    assert int((got != fx['expected']).sum()) == 0 and got.sum() == 13548


@pytest.mark.parametrize('shape,kind', [((4, 128, 200), 'channel'), ((2, 3, 5, 7, 37), 'channel'),
                                        ((3, 70, 129), 'shared'), ((2, 64, 1), 'channel')])
def test_res_bwd(slayer, shape, kind):
    gen = torch.Generator().manual_seed(seed_of(shape, kind, 'resb'))
    f = lambda: torch.randn(shape, generator=gen)
    g_re, g_im, re, im = f(), f(), f(), f()
    sin, cos = _rot(kind, shape, gen)
    ref = O.res_bwd(g_re, g_im, re, im, sin, cos)
    from lava_dl_amd.slayer.neuron.dynamics import resonator as R
    got = R._bwd(g_re.to(dev()), g_im.to(dev()), re.to(dev()), im.to(dev()), sin.to(dev()), cos.to(dev()))
    assert_exact(got[0], ref[0], 'res_bwd grad_real_input')
    assert_exact(got[1], ref[1], 'res_bwd grad_imag_input')
    s_sum, s_mag, c_sum, c_mag = res_decay_grads_f64(got[0], got[1], re, im, sin.numel())
    assert_sum(got[2], s_sum, s_mag, 'res_bwd grad_sin')
    assert_sum(got[3], c_sum, c_mag, 'res_bwd grad_cos')


def test_res_autograd_and_nan_guard(slayer):
    gen = torch.Generator().manual_seed(31)
    shape = (2, 8, 50)
    xr = sparse_input(gen, shape, p=0.3).to(dev()).requires_grad_()
    xi = sparse_input(gen, shape, p=0.3).to(dev()).requires_grad_()
    sin = torch.full((8,), 2103.0, device=dev(), requires_grad=True)
    cos = torch.full((8,), 3273.0, device=dev(), requires_grad=True)
    zero = torch.tensor([0.0], device=dev())
    re, im = slayer.neuron.dynamics.resonator.dynamics(xr, xi, sin, cos, zero, zero, 64)
    (re.sum() + 2 * im.sum()).backward()
    ref = O.res_bwd(torch.ones(shape), 2 * torch.ones(shape), re.detach().cpu(), im.detach().cpu(),
                    sin.detach().cpu(), cos.detach().cpu())
    assert_exact(xr.grad, ref[0], 'res autograd grad_real')
    assert_exact(xi.grad, ref[1], 'res autograd grad_imag')
    assert_rel(sin.grad, ref[2], 'res autograd grad_sin')
    assert_rel(cos.grad, ref[3], 'res autograd grad_cos')
    re, im = slayer.neuron.dynamics.resonator.dynamics(xr, xi, sin, cos, zero, zero, 64)
    bad = torch.ones(shape, device=dev())
    bad[0, 0, 10] = float('nan')
    with pytest.raises(Exception):
        torch.autograd.backward([re, im], [bad, torch.ones(shape, device=dev())])


# ------------------------------------------------------------------------- APTH / adaptive RES
@pytest.mark.parametrize('shape,kind,w', [((4, 128, 200), 'channel', 64), ((2, 3, 5, 7, 37), 'channel', 4096),
                                          ((3, 70, 129), 'neuron', 100), ((4, 9000, 100), 'channel', 64),
                                          ((4, 35000, 40), 'channel', 64), ((1, 5, 3), 'shared', 64)])
def test_apth_and_adres_bit_exact(slayer, shape, kind, w):
    gen = torch.Generator().manual_seed(seed_of(shape, kind, w, 'apth'))
    xr = sparse_input(gen, shape, p=0.4, amp=3.0)
    xi = torch.randn(shape, generator=gen)
    rd, td = _decay(kind, shape, gen), _decay(kind, shape, gen)
    sin, cos = _rot(kind, shape, gen)
    st = lambda: torch.randn(shape[:-1], generator=gen)
    ims, refs, ths, res = st(), st(), st() + 1.5, st()
    D = slayer.neuron.dynamics
    g = lambda t: t.to(dev())
    r_th, r_ref = O.apth_fwd(xr, xi, ims, refs, rd, ths, td, 0.5, 1.0, w)
    th, ref = D.adaptive_phase_th.dynamics(g(xr), g(xi), g(ims), g(refs), g(rd), g(ths), g(td), 0.5, 1.0, w)
    assert_exact(th, r_th, f'apth threshold {shape}')
    assert_exact(ref, r_ref, f'apth refractory {shape}')
    want = O.adres_fwd(xr, xi, sin, cos, rd, td, res, ims, refs, ths, 0.5, 1.0, w)
    got = D.adaptive_resonator.dynamics(g(xr), g(xi), g(sin), g(cos), g(rd), g(td), g(res), g(ims), g(refs),
                                        g(ths), 0.5, 1.0, w)
    for a, b, name in zip(got, want, ('real', 'imag', 'threshold', 'refractory')):
        assert_exact(a, b, f'adres {name} {shape}')


def test_adres_autograd(slayer):
    gen = torch.Generator().manual_seed(91)
    shape = (2, 8, 60)
    xr = sparse_input(gen, shape, p=0.3).to(dev()).requires_grad_()
    xi = sparse_input(gen, shape, p=0.3).to(dev()).requires_grad_()
    sin = torch.full((8,), 2103.0, device=dev(), requires_grad=True)
    cos = torch.full((8,), 3273.0, device=dev(), requires_grad=True)
    d = torch.full((8,), 200.0, device=dev())
    zero, one = torch.zeros(1, device=dev()), torch.ones(1, device=dev())
    re, im, th, ref = slayer.neuron.dynamics.adaptive_resonator.dynamics(xr, xi, sin, cos, d, d, zero, zero, zero,
                                                                         one, 0.5, 1.0, 64)
    assert not th.requires_grad and not ref.requires_grad
    (re.sum() + 2 * im.sum()).backward()
    want = O.res_bwd(torch.ones(shape), 2 * torch.ones(shape), re.detach().cpu(), im.detach().cpu(),
                     sin.detach().cpu(), cos.detach().cpu())
    assert_exact(xr.grad, want[0], 'adres grad real')
    assert_exact(xi.grad, want[1], 'adres grad imag')
    assert_rel(sin.grad, want[2], 'adres grad sin')
    assert_rel(cos.grad, want[3], 'adres grad cos')


# --------------------------------------------------------------------------------- debug mode
def test_debug_mode_cross_check_passes_and_catches_overflow(slayer):
    """debug=True runs the independent one-thread-per-neuron kernels (64-bit state) next to the
    streaming kernels: silent when they agree, an exception when a state leaves the 32-bit range."""
    gen = torch.Generator().manual_seed(77)
    shape = (2, 40, 132)
    x = sparse_input(gen, shape, p=0.3, amp=2.0).to(dev()).requires_grad_()
    x2 = sparse_input(gen, shape, p=0.3, amp=2.0).to(dev()).requires_grad_()
    d = torch.randint(0, 4097, (40,), generator=gen).float().to(dev()).requires_grad_()
    zero, one = torch.zeros(1, device=dev()), torch.ones(1, device=dev())
    D = slayer.neuron.dynamics
    y = D.leaky_integrator.dynamics(x, d, zero, 64, 1.0, debug=True)
    ref = O.li_fwd(x.detach().cpu(), d.detach().cpu(), torch.tensor([0.0]), 64, 1.0)
    assert_exact(y, ref, 'debug li_fwd')
    y.sum().backward()
    D.adaptive_threshold.dynamics(x.detach(), zero, d.detach(), one, d.detach(), 0.5, 1.0, 64, debug=True)
    for thr in (None, 1.5):
        re, im = D.resonator.dynamics(x, x2, (d * 0.5).round(), (d * 0.6).round(), zero, zero, 64, thr, debug=True)
        (re.sum() + im.sum()).backward()
    # an integrator (decay 0) driven beyond 2^31: the 32-bit streaming state saturates/wraps, the check fires
    big = torch.full((1, 1, 64), 3.0e7, device=dev())
    # (or the kernel's own range check does, when its report reaches the host before the comparison is made)
    with pytest.raises(Exception, match='implementations differ|32-bit range'):
        D.leaky_integrator.dynamics(big, zero, zero, 64, debug=True)
    torch.cuda.synchronize()
    slayer.clear_range_flag()
    # the naive kernel itself follows the int64 oracle there
    from lava_dl_amd.slayer.neuron.dynamics import leaky_integrator as L
    got = L._fwd(big, zero, zero, -1, 64, entry='slayer_li_fwd_naive')
    assert_exact(got, O.li_fwd(big.cpu(), torch.tensor([0.0]), torch.tensor([0.0]), 64), 'naive li_fwd beyond 2^31')


def test_rows_longer_than_the_vector_path_allows(slayer):
    """T > 2**22 leaves the dwordx4 kernels (32-bit byte offsets per wave) for the dword kernel;
    too long for the CPU oracle, so the independent one-thread-per-neuron kernel is the checker
    (debug=True raises on any mismatch) and the head of the rows is compared with the oracle."""
    gen = torch.Generator().manual_seed(77)
    T = (1 << 22) + 8
    x = sparse_input(gen, (1, 3, T), p=0.05, amp=1.5).to(dev()).requires_grad_()
    d = torch.tensor([300.0, 1000.0, 4000.0], device=dev(), requires_grad=True)
    zero = torch.zeros(1, device=dev())
    y = slayer.neuron.dynamics.leaky_integrator.dynamics(x, d, zero, 64, 1.0, debug=True)
    y.backward(torch.ones_like(y) * 1e-3)
    head = 2048
    ref = O.li_fwd(x.detach().cpu()[..., :head], d.detach().cpu(), torch.tensor([0.0]), 64, 1.0)
    assert_exact(y.detach()[..., :head], ref, 'li_fwd long rows, head')
    assert torch.isfinite(x.grad).all() and float(x.grad.abs().sum()) > 0


def test_two_streams_and_two_threads(slayer):
    """Entry points take the caller's stream and keep no per-call global state: launches from two
    host threads on two streams, interleaved, give the same bits as serial launches."""
    import threading
    gen = torch.Generator().manual_seed(91)
    shapes = [(4, 64, 33, 300), (2, 40, 17, 128)]
    xs = [sparse_input(gen, s, p=0.2, amp=1.5).to(dev()) for s in shapes]
    ds = [torch.randint(0, 4096, (s[1],), generator=gen).float().to(dev()) for s in shapes]
    zero = torch.zeros(1, device=dev())
    D = slayer.neuron.dynamics.leaky_integrator
    want = [D.dynamics(x, d, zero, 64, 1.0) for x, d in zip(xs, ds)]
    torch.cuda.synchronize()
    got, errors = [None, None], []

    def work(i):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for _ in range(20):
                    y = D.dynamics(xs[i], ds[i], zero, 64, 1.0)
                stream.synchronize()
            got[i] = y
        except Exception as e:      # surfaced in the main thread below
            errors.append(e)

    threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for i in range(2):
        assert torch.equal(got[i], want[i]), f'stream {i}: result differs from the serial launch'
