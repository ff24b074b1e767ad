"""The float backward recurrences as wave scans (csrc/scan.hip: tensors of 2^20 elements and more) against the
oracle's step-by-step loops (neuron/dynamics/leaky_integrator.py:234-259, resonator.py:379-467 in the reference)
and against the one-thread-per-neuron GPU kernels; the fused CUBA / ALIF backward scans against the chain of
spike backward + two leaky-integrator scans, bit for bit."""
import pytest
import torch

from oracle import slayer_oracle as O
from tests.util import (dev, sparse_input, assert_rel, assert_scale, assert_sum, li_bwd_f64, li_decay_grad_f64,
                        res_decay_grads_f64, seed_of, SCAN_MIN)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope='module')
def slayer():
    import lava_dl_amd.slayer as s
    return s


# (shape, number of decays): rows of one quad, rows shorter / longer than a wave and than a pass, row counts that
# do not fill the last workgroup, rows that are a whole number of lines and rows that are not, per-neuron decays
SHAPES = [((262144 + 3, 1, 4), 1), ((3, 43691, 8), 43691), ((5, 1024, 300), 1024), ((2, 4099, 128), 4099),
          ((7, 161, 1000), 161), ((3, 43, 8196), 43), ((1, 2, 524288), 2), ((2, 16, 33, 31, 76), 16),
          # rows that are not a whole number of quads (T % 4 = 1, 2, 3): the any-length form of the scans
          ((5, 1024, 301), 1024), ((7, 161, 1002), 161), ((3, 43, 8195), 43), ((2, 4099, 129), 4099),
          ((4, 4100, 67), 4100), ((1, 3, 400001), 3)]


@pytest.mark.parametrize('shape,nd', SHAPES)
def test_li_bwd_scan_against_oracle_and_sequential_kernel(slayer, shape, nd):
    L = slayer.neuron.dynamics.leaky_integrator
    gen = torch.Generator().manual_seed(seed_of('li-scan', shape))
    numel = 1
    for s in shape:
        numel *= s
    assert numel >= SCAN_MIN
    g = torch.randn(shape, generator=gen)
    y = torch.randn(shape, generator=gen) * 2
    d = torch.randint(0, 4097, (nd,), generator=gen).float()
    d[0] = 0.0                                     # a pure integrator: the longest carries
    if nd > 1:
        d[1] = 4096.0                              # nothing carried at all
    gi, gd = L._bwd(g.to(dev()), y.to(dev()), d.to(dev()))
    seq = L._bwd_naive(g.to(dev()), d.to(dev()))
    # two float32 evaluations of the same recurrence: within 1e-5 of the largest value while the rows are short
    # enough for that to be a meaningful scale; on the rows of several hundred thousand steps a pure integrator is a
    # random walk whose terms sum to a thousand times its largest value, and the bar is the one against float64 below
    long_rows = shape[-1] > 65536
    if not long_rows:
        assert_scale(gi, seq.cpu(), 'scan vs step-by-step kernel')
    # the oracle on slabs of rows (whole tensor when it is small enough for the python loop over time)
    rows = g.reshape(-1, shape[-1])
    M = rows.shape[0]
    npb = M // shape[0]
    pick = torch.unique(torch.cat([torch.arange(0, min(M, 40)), torch.arange(max(M - 40, 0), M),
                                   torch.randint(0, M, (60,), generator=gen)]))
    idx = ((pick % npb) // (npb // nd)) if nd > 1 else torch.zeros_like(pick)
    a = (1 - d[idx] / 4096).reshape(-1, 1)
    go, ref = rows[pick], torch.zeros(len(pick), shape[-1])
    acc = torch.zeros(len(pick), 1)
    for t in range(shape[-1] - 1, -1, -1):
        acc = a * acc + go[:, t:t + 1]
        ref[:, t:t + 1] = acc
    want64, mag64 = li_bwd_f64(go, a.float())          # every element against the magnitudes of its own terms
    got = gi.reshape(-1, shape[-1])[pick.to(dev())]
    assert_sum(got, want64, mag64, 'scan vs float64 recurrence, elementwise')
    if long_rows:
        assert_sum(seq.reshape(-1, shape[-1])[pick.to(dev())], want64, mag64, 'step-by-step kernel vs float64 recurrence')
        assert_sum(ref, want64, mag64, 'step-by-step recurrence (float32) vs float64 recurrence')
    else:
        assert_scale(got, ref, 'scan vs step-by-step recurrence (float32)')
    # decay gradient in float64 from the sequential result
    assert_sum(gd, *li_decay_grad_f64(seq, y, nd), 'grad_decay')


def test_li_bwd_scan_whole_tensor_against_oracle(slayer):
    L = slayer.neuron.dynamics.leaky_integrator
    shape = (4, 16, 64, 300)
    gen = torch.Generator().manual_seed(77)
    g, y = torch.randn(shape, generator=gen), torch.randn(shape, generator=gen)
    d = torch.randint(0, 4096, (16,), generator=gen).float()
    gi, gd = L._bwd(g.to(dev()), y.to(dev()), d.to(dev()))
    r_gi, r_gd = O.li_bwd(g, y, d)
    assert_scale(gi, r_gi, 'grad_input vs oracle')
    assert_rel(gd, r_gd, 'grad_decay vs oracle')


@pytest.mark.parametrize('shape,nd', [((3, 700, 520), 700), ((2, 16, 40, 32, 28), 16), ((9, 128, 1000), 1),
                                      ((3, 700, 521), 700), ((9, 128, 1003), 1), ((6, 300, 602), 300)])
def test_res_bwd_scan_against_oracle(slayer, shape, nd):
    R = slayer.neuron.dynamics.resonator
    gen = torch.Generator().manual_seed(seed_of('res-scan', shape))
    g_re, g_im = torch.randn(shape, generator=gen), torch.randn(shape, generator=gen)
    re, im = torch.randn(shape, generator=gen), torch.randn(shape, generator=gen)
    decay = torch.randint(40, 4096, (nd,), generator=gen).float()
    phi = 2 * 3.141592653589793 * torch.rand(nd, generator=gen)
    sin, cos = ((4096 - decay) * torch.sin(phi)).round(), ((4096 - decay) * torch.cos(phi)).round()
    to = lambda t: t.to(dev())
    got = R._bwd(to(g_re), to(g_im), to(re), to(im), to(sin), to(cos))
    n = min(shape[0], 2)
    want = O.res_bwd(g_re[:n], g_im[:n], re[:n], im[:n], sin, cos)
    assert_scale(got[0][:n], want[0], 'grad real')
    assert_scale(got[1][:n], want[1], 'grad imag')
    seq = R._bwd_naive(to(g_re), to(g_im), to(sin), to(cos)) if hasattr(R, '_bwd_naive') else None
    if seq is not None:
        assert_scale(got[0], seq[0].cpu(), 'grad real vs step-by-step kernel')
        assert_scale(got[1], seq[1].cpu(), 'grad imag vs step-by-step kernel')
        s_sum, s_mag, c_sum, c_mag = res_decay_grads_f64(seq[0], seq[1], re, im, nd)
        assert_sum(got[2], s_sum, s_mag, 'grad sin')
        assert_sum(got[3], c_sum, c_mag, 'grad cos')


@pytest.mark.parametrize('shape', [(5, 1024, 300), (2, 16, 33, 31, 76), (3, 43, 8196),
                                   (5, 1024, 301), (3, 43, 8194), (4, 2100, 127)])
@pytest.mark.parametrize('graded', [False, True])
@pytest.mark.parametrize('kind', ['cuba', 'alif'])
def test_fused_backward_scans_equal_the_chain_of_scans_bit_for_bit(slayer, shape, graded, kind):
    """Same arithmetic, same spans: spike backward + leaky-integrator scan (voltage) + leaky-integrator scan
    (current) and the one fused kernel give the same input gradient, every bit."""
    D = slayer.neuron.dynamics
    S = slayer.spike.spike
    gen = torch.Generator().manual_seed(seed_of('fused-scan', shape, graded, kind))
    C = shape[1]
    g = torch.randn(shape, generator=gen).to(dev())
    vol = (torch.randn(shape, generator=gen) * 1.5).to(dev())
    cur = torch.randn(shape, generator=gen).to(dev())
    theta = (1 + torch.rand(shape, generator=gen)).to(dev())
    di = torch.randint(0, 4097, (C,), generator=gen).float().to(dev())
    dv = torch.randint(0, 4097, (C,), generator=gen).float().to(dev())
    thr, tau, rho = 1.0, 0.7, 1.3
    for need in (True, False):
        if kind == 'cuba':
            gx, g_i, g_v = D.cuba_fused._bwd(g, vol, cur if need else None, di, dv, thr, tau, rho, graded, need)
            gv = S._bwd(g, vol, None, thr, tau, rho, graded)
        else:
            gx, g_i, g_v = D.alif_fused._bwd(g, vol, theta, cur if need else None, di, dv, tau, rho, graded, need)
            gv = S._bwd(g, vol, theta, 0.0, tau, rho, graded)
        gc, r_gv = D.leaky_integrator._bwd(gv, vol, dv, need)
        r_gx, r_gi = D.leaky_integrator._bwd(gc, cur, di, need)
        assert torch.equal(gx, r_gx), f'{kind} fused scan differs from the chain (decay gradients: {need})'
        if need:
            assert_rel(g_i, r_gi.cpu(), 'grad current decay')
            assert_rel(g_v, r_gv.cpu(), 'grad voltage decay')


@pytest.mark.parametrize('shape', [(5, 1024, 300), (2, 16, 33, 31, 76), (3, 43, 8196),
                                   (5, 1024, 301), (3, 43, 8194), (4, 2100, 127)])
@pytest.mark.parametrize('graded', [False, True])
def test_fused_rf_backward_scan_equals_the_chain_of_scans_bit_for_bit(slayer, shape, graded):
    """Complex spike surrogate + resonator backward scan in one kernel against the two operators in a row (same
    arithmetic, same spans), and the surrogate + oracle loop on a slab."""
    D = slayer.neuron.dynamics
    C = slayer.spike.complex
    gen = torch.Generator().manual_seed(seed_of('rf-scan', shape, graded))
    n = shape[1]
    g = torch.randn(shape, generator=gen).to(dev())
    re = (torch.randn(shape, generator=gen) * 1.5).to(dev())
    im = torch.randn(shape, generator=gen).to(dev())
    decay = torch.randint(40, 4096, (n,), generator=gen).float()
    phi = 2 * 3.141592653589793 * torch.rand(n, generator=gen)
    sin = ((4096 - decay) * torch.sin(phi)).round().to(dev())
    cos = ((4096 - decay) * torch.cos(phi)).round().to(dev())
    thr, tau, rho = 1.0, 0.7, 1.3
    for need in (True, False):
        g_re, g_im, g_sin, g_cos = D.rf_fused._bwd(g, re, im, sin, cos, thr, tau, rho, graded, need)
        s_re, s_im = C._bwd(g, re, im, None, thr, tau, rho, graded)
        r_re, r_im, r_sin, r_cos = D.resonator._bwd(s_re, s_im, re, im, sin, cos, need)
        assert torch.equal(g_re, r_re) and torch.equal(g_im, r_im), f'fused RF scan differs from the chain ({need})'
        if need:
            assert_rel(g_sin, r_sin.cpu(), 'grad sin')
            assert_rel(g_cos, r_cos.cpu(), 'grad cos')
    k = min(shape[0], 2)
    o_re, o_im = O.cspike_bwd(g[:k].cpu(), re[:k].cpu(), im[:k].cpu(), thr, tau, rho, graded)
    want = O.res_bwd(o_re, o_im, re[:k].cpu(), im[:k].cpu(), sin.cpu(), cos.cpu())
    assert_scale(g_re[:k], want[0], 'grad real vs oracle')
    assert_scale(g_im[:k], want[1], 'grad imag vs oracle')


@pytest.mark.parametrize('shape', [(5, 1024, 300), (3, 43, 8196), (5, 1024, 301)])
@pytest.mark.parametrize('bad', [float('nan'), float('inf')])
def test_a_non_finite_row_does_not_reach_its_neighbours(slayer, shape, bad):
    """Rows are independent in the step-by-step recurrences (neuron/dynamics/leaky_integrator.py:234-259,
    resonator.py:379-467 in the reference): a NaN or Inf in the gradient of one row must leave every other row of
    the scan's span exactly as it is without it -- the cut at a row end lets nothing in, not 0 * Inf either."""
    D = slayer.neuron.dynamics
    gen = torch.Generator().manual_seed(seed_of('scan-nonfinite', shape))
    C, T = shape[1], shape[-1]
    g = torch.randn(shape, generator=gen)
    y = torch.randn(shape, generator=gen)
    cur = torch.randn(shape, generator=gen)
    d = torch.randint(0, 4097, (C,), generator=gen).float()
    d2 = torch.randint(0, 4097, (C,), generator=gen).float()
    rows = g.reshape(-1, T)
    M = rows.shape[0]
    victims = [3, M // 2 + 1, M - 2]                     # inside a span, wherever spans happen to begin and end
    dirty = rows.clone()
    for i, r in enumerate(victims):
        dirty[r, (T // 3) * (i + 1) - 1 if i < 2 else T - 1] = bad
    dirty = dirty.reshape(shape)
    clean_rows = torch.ones(M, dtype=torch.bool)
    clean_rows[victims] = False
    to = lambda t: t.to(dev())

    def untouched(a, b, what):
        a, b = a.reshape(-1, T)[clean_rows.to(a.device)], b.reshape(-1, T)[clean_rows.to(b.device)]
        assert bool(torch.isfinite(a).all()), what + ': a clean row became non-finite'
        assert torch.equal(a, b), what + ': a clean row changed'

    want, _ = D.leaky_integrator._bwd(to(g), to(y), to(d), True)
    got, _ = D.leaky_integrator._bwd(to(dirty), to(y), to(d), True)
    untouched(got, want, 'leaky integrator scan')
    assert not bool(torch.isfinite(got.reshape(-1, T)[victims]).all())

    sin = ((4096 - d.clamp(40, 4095)) * 0.6).round()
    cos = ((4096 - d.clamp(40, 4095)) * 0.8).round()
    want = D.resonator._bwd(to(g), to(cur), to(y), to(cur), to(sin), to(cos), True)
    got = D.resonator._bwd(to(dirty), to(cur), to(y), to(cur), to(sin), to(cos), True)
    untouched(got[0], want[0], 'resonator scan, real')
    untouched(got[1], want[1], 'resonator scan, imag')

    want = D.cuba_fused._bwd(to(g), to(y), to(cur), to(d), to(d2), 1.0, 0.7, 1.3, False, True)[0]
    got = D.cuba_fused._bwd(to(dirty), to(y), to(cur), to(d), to(d2), 1.0, 0.7, 1.3, False, True)[0]
    untouched(got, want, 'fused CUBA scan')
