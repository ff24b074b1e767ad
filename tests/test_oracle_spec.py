"""Pins for the parts of the oracle that no reference-held fixture reaches:
brute force against the scalar big-int spec, closed forms, and independent
library routines (torch autograd, scipy.signal.lfilter, numpy.convolve,
numpy slicing).  The invariants mirror the reference's own unit tests
(tests/lava/lib/dl/slayer/neuron/dynamics/test_*.py, utils/time/test_shift.py,
utils/filter/test_conv_filter.py)."""
import itertools

import numpy as np
import pytest
import scipy.signal
import torch

from oracle import scalar_spec as S
from oracle import slayer_oracle as O

DECAYS = [0.0, 1.0, 2047.0, 4095.0, 4096.0, 1234.7]


def _rand_input(rng, shape, p=0.3, amp=3.0):
    x = rng.standard_normal(shape) * amp * (rng.random(shape) < p)
    return torch.tensor(x, dtype=torch.float32)


# ---------------------------------------------------------------- LI forward
@pytest.mark.parametrize('w', [64, 4096, 100])
@pytest.mark.parametrize('thr', [None, 1.25, 0.5001])
def test_li_fwd_matches_scalar_spec(w, thr):
    rng = np.random.default_rng(10 + w)
    T = 40
    x = _rand_input(rng, (2, len(DECAYS), T))
    decay = torch.tensor(DECAYS)
    state = torch.tensor(rng.standard_normal((2, len(DECAYS))) * 2, dtype=torch.float32)
    out = O.li_fwd(x, decay, state, w, thr)
    for n, c in itertools.product(range(2), range(len(DECAYS))):
        ref, _ = S.li(x[n, c].tolist(), DECAYS[c], float(state[n, c]), w, thr)
        assert np.array_equal(out[n, c].numpy(), np.array(ref, dtype=np.float32)), (n, c)


def test_li_fwd_closed_forms():
    rng = np.random.default_rng(3)
    x = _rand_input(rng, (3, 4, 50))
    w = 64
    u = torch.trunc(x * w)
    zero = torch.tensor([0.0])
    # decay 4096 -> nothing is carried over
    assert torch.equal(O.li_fwd(x, torch.tensor([4096.0]), zero, w), u / w)
    # decay 0, no threshold -> running sum
    assert torch.equal(O.li_fwd(x, zero, zero, w), torch.cumsum(u, -1) / w)
    # one impulse: k-fold truncated multiplication, both signs
    for amp in (1000.0, -1000.0):
        imp = torch.zeros(1, 1, 30)
        imp[..., 0] = amp
        y = O.li_fwd(imp, torch.tensor([300.0]), zero, w)
        v = int(amp * w)
        for k in range(30):
            assert y[0, 0, k].item() * w == v
            v = S.trunc_div_4096(v * (4096 - 300))


def test_li_threshold_edge_and_reset():
    w = 64
    zero = torch.tensor([0.0])
    # state exactly at threshold*w fires; one below does not (integer threshold)
    x = torch.tensor([[[2.0, 0.0, 0.0]], [[2.0 - 1 / 64, 0.0, 0.0]]])
    y = O.li_fwd(x, zero, zero, w, threshold=2.0)
    assert y[0, 0].tolist() == [2.0, 0.0, 0.0]
    assert y[1, 0].tolist() == [2.0 - 1 / 64] * 3
    # fractional scaled threshold: 5120.01 behaves as >= 5121 (eps of the neuron classes)
    x = torch.tensor([[[1.25, 0.0]], [[1.25 + 1 / 4096, 0.0]]])
    y = O.li_fwd(x, zero, zero, 4096, threshold=1.25 + 0.01 / 4096)
    assert y[0, 0, 1].item() == 1.25 and y[1, 0, 1].item() == 0.0
    # threshold 0 disables the reset on this path (leaky_integrator.py:223)
    x = torch.tensor([[[1.0, 1.0]]])
    assert O.li_fwd(x, zero, zero, w, threshold=0.0)[0, 0].tolist() == [1.0, 2.0]


def test_li_integer_states_and_batch_consistency():
    rng = np.random.default_rng(5)
    x = _rand_input(rng, (1, 6, 80)).repeat(4, 1, 1)
    w = 1 << 12
    y = O.li_fwd(x, torch.tensor([777.0]), torch.tensor([0.0]), w, threshold=1.0)
    assert torch.equal(torch.floor(y * w), y * w)
    assert float(y.var(dim=0).max()) == 0.0


def test_li_split_invariance():
    """Carrying the last state across a time split gives the same trace
    (the reference's persistent-state test, tests/.../neuron/test_cuba.py:136-271)."""
    rng = np.random.default_rng(6)
    x = _rand_input(rng, (2, 5, 60))
    decay = torch.tensor([100.0, 900.0, 0.0, 4095.0, 2222.0])
    w, thr = 64, 1.5
    full = O.li_fwd(x, decay, torch.tensor([0.0]), w, thr)
    a = O.li_fwd(x[..., :23], decay, torch.tensor([0.0]), w, thr)
    st = O.li_persistent_state(a[..., -1], O.spike_fwd(a[..., -1], thr))
    b = O.li_fwd(x[..., 23:], decay, st, w, thr)
    assert torch.equal(torch.cat([a, b], -1), full)


def test_per_channel_decay_on_spatial_tensor():
    rng = np.random.default_rng(7)
    x = _rand_input(rng, (2, 3, 4, 5, 20))
    decay = torch.tensor([0.0, 500.0, 4000.0])
    y = O.li_fwd(x, decay, torch.tensor([0.0]), 64)
    for c in range(3):
        yc = O.li_fwd(x[:, c].reshape(2, 20, 20), decay[c:c + 1], torch.tensor([0.0]), 64)
        assert torch.equal(y[:, c].reshape(2, 20, 20), yc)


# --------------------------------------------------------------- LI backward
def test_li_bwd_is_adjoint_of_float_iir():
    rng = np.random.default_rng(8)
    N, C, T = 3, 4, 37
    go = torch.tensor(rng.standard_normal((N, C, T)), dtype=torch.float32)
    out = torch.tensor(rng.standard_normal((N, C, T)), dtype=torch.float32)
    decay = torch.tensor([0.0, 100.0, 2048.0, 4000.0])
    g, gd = O.li_bwd(go, out, decay)
    # float64 lfilter on the reversed sequence
    a = 1 - decay.double().numpy() / 4096
    for c in range(C):
        ref = scipy.signal.lfilter([1.0], [1.0, -a[c]], go[:, c].double().numpy()[:, ::-1], axis=-1)[:, ::-1]
        assert np.allclose(g[:, c].numpy(), ref, rtol=1e-5, atol=1e-5)
    # autograd through y[t] = a*y[t-1] + x[t]; d/da uses the saved (here: arbitrary) output trace
    av = torch.tensor(a, dtype=torch.float64, requires_grad=True)
    x = torch.zeros(N, C, T, dtype=torch.float64, requires_grad=True)
    ys, y = [], torch.zeros(N, C, dtype=torch.float64)
    for t in range(T):
        y = av * y + x[..., t]
        ys.append(y)
    (torch.stack(ys, -1) * go.double()).sum().backward()
    assert np.allclose(g.numpy(), x.grad.numpy(), rtol=1e-5, atol=1e-5)
    ref_gd = (g.double()[..., 1:] * out.double()[..., :-1]).sum(dim=(0, 2))
    assert np.allclose(gd.numpy(), ref_gd.numpy(), rtol=1e-5, atol=1e-5)
    # shared decay -> one number
    g1, gd1 = O.li_bwd(go, out, torch.tensor([100.0]))
    assert gd1.shape == (1,)
    assert np.isclose(gd1.item(), (g1.double()[..., 1:] * out.double()[..., :-1]).sum().item(), rtol=1e-5)


def test_li_bwd_true_parameter_gradient():
    """With out = the float IIR's own output, grad_decay is d loss / d a."""
    rng = np.random.default_rng(9)
    T = 25
    x = torch.tensor(rng.standard_normal((2, 1, T)), dtype=torch.float64)
    go = torch.tensor(rng.standard_normal((2, 1, T)), dtype=torch.float64)
    a = torch.tensor([0.8], dtype=torch.float64, requires_grad=True)
    y, ys = torch.zeros(2, 1, dtype=torch.float64), []
    for t in range(T):
        y = a * y + x[..., t]
        ys.append(y)
    out = torch.stack(ys, -1)
    (out * go).sum().backward()
    _, gd = O.li_bwd(go.float(), out.detach().float(), torch.tensor([(1 - 0.8) * 4096]))
    assert np.isclose(gd.item(), a.grad.item(), rtol=1e-4)


# ----------------------------------------------------------------------- ATH
@pytest.mark.parametrize('w', [64, 4096])
def test_ath_matches_scalar_spec(w):
    rng = np.random.default_rng(20 + w)
    T, C = 60, len(DECAYS)
    x = _rand_input(rng, (2, C, T), p=0.5, amp=2.0)
    rd = torch.tensor(DECAYS)
    td = torch.tensor(DECAYS[::-1])
    th_state = torch.tensor(rng.random((2, C)) * 2, dtype=torch.float32)    # includes th < th0
    ref_state = torch.tensor(rng.standard_normal((2, C)), dtype=torch.float32)  # includes r < 0
    th, ref = O.ath_fwd(x, ref_state, rd, th_state, td, 0.5, 1.0, w)
    for n, c in itertools.product(range(2), range(C)):
        t_ref, r_ref, _ = S.ath(x[n, c].tolist(), float(ref_state[n, c]), DECAYS[c],
                                float(th_state[n, c]), DECAYS[::-1][c], 0.5, 1.0, w)
        assert np.array_equal(th[n, c].numpy(), np.array(t_ref, dtype=np.float32))
        assert np.array_equal(ref[n, c].numpy(), np.array(r_ref, dtype=np.float32))


def test_ath_closed_forms():
    w = 64
    x = torch.zeros(1, 1, 20)
    one = torch.tensor([1.0])
    # no input above threshold: threshold relaxes to th0 from above, refractory to 0
    th, ref = O.ath_fwd(x - 5, torch.tensor([2.0]), torch.tensor([1000.0]), torch.tensor([3.0]),
                        torch.tensor([1000.0]), 0.5, 1.0, w)
    t, r = 3 * w, 2 * w
    for k in range(20):
        r = S.trunc_div_4096(r * 3096)
        t = S.trunc_div_4096((t - w) * 3096) + w
        assert th[0, 0, k].item() * w == t and ref[0, 0, k].item() * w == r
    # a spike adds step to the threshold and 2*threshold to the refractory state
    x = torch.zeros(1, 1, 3)
    x[..., 0] = 10.0
    th, ref = O.ath_fwd(x, torch.tensor([0.0]), torch.tensor([0.0]), one, torch.tensor([0.0]), 0.5, 1.0, w)
    assert th[0, 0].tolist() == [1.0, 1.5, 1.5]
    assert ref[0, 0].tolist() == [0.0, 2.0, 2.0]


def test_apth_matches_scalar_spec_and_its_parts():
    rng = np.random.default_rng(25)
    T, C, w = 80, len(DECAYS), 64
    xr = _rand_input(rng, (2, C, T), p=0.6, amp=3.0)
    xi = torch.tensor(rng.standard_normal((2, C, T)), dtype=torch.float32)
    rd, td = torch.tensor(DECAYS), torch.tensor(DECAYS[::-1])
    th_state = torch.tensor(rng.random((2, C)) * 2, dtype=torch.float32)
    ref_state = torch.tensor(rng.standard_normal((2, C)), dtype=torch.float32)
    im_state = torch.tensor(rng.standard_normal((2, C)), dtype=torch.float32)
    th, ref = O.apth_fwd(xr, xi, im_state, ref_state, rd, th_state, td, 0.5, 1.0, w)
    spikes = 0
    for n, c in itertools.product(range(2), range(C)):
        t_ref, r_ref, fired = S.apth(xr[n, c].tolist(), xi[n, c].tolist(), float(im_state[n, c]),
                                     float(ref_state[n, c]), DECAYS[c], float(th_state[n, c]),
                                     DECAYS[::-1][c], 0.5, 1.0, w)
        spikes += sum(fired)
        assert np.array_equal(th[n, c].numpy(), np.array(t_ref, dtype=np.float32))
        assert np.array_equal(ref[n, c].numpy(), np.array(r_ref, dtype=np.float32))
    assert spikes > 0
    # with an imaginary part that always crosses zero upwards the op reduces to ath_fwd on the real part
    zig = torch.ones(2, C, T)
    zig[..., ::2] = -1.0
    up = torch.cat([-torch.ones(2, C, 1), zig[..., :-1]], -1)        # previous sample of each step
    only_up = (zig >= 0) & (up < 0)
    th_a, ref_a = O.apth_fwd(torch.where(only_up, xr, torch.full_like(xr, -100.0)), zig, -torch.ones(2, C),
                             ref_state, rd, th_state, td, 0.5, 1.0, w)
    th_b, ref_b = O.ath_fwd(torch.where(only_up, xr, torch.full_like(xr, -100.0)), ref_state, rd, th_state, td,
                            0.5, 1.0, w)
    assert torch.equal(th_a, th_b) and torch.equal(ref_a, ref_b)


def test_adres_matches_scalar_spec_and_its_parts():
    rng = np.random.default_rng(26)
    T, w = 70, 64
    sin = [2103.0, 1.0, 3000.5, -2000.0]
    cos = [3273.0, 4095.0, 0.0, 2500.0]
    rdl, tdl = [0.0, 100.0, 4096.0, 2000.0], [4095.0, 50.0, 0.0, 1234.0]
    C = len(sin)
    xr, xi = _rand_input(rng, (2, C, T)), _rand_input(rng, (2, C, T))
    st = lambda: torch.tensor(rng.standard_normal((2, C)), dtype=torch.float32)
    rs, is_, refs, ths = st(), st(), st(), st() + 1.5
    outs = O.adres_fwd(xr, xi, torch.tensor(sin), torch.tensor(cos), torch.tensor(rdl), torch.tensor(tdl),
                       rs, is_, refs, ths, 0.5, 1.0, w)
    spikes = 0
    for n, c in itertools.product(range(2), range(C)):
        ref = S.adres(xr[n, c].tolist(), xi[n, c].tolist(), sin[c], cos[c], rdl[c], tdl[c],
                      float(rs[n, c]), float(is_[n, c]), float(refs[n, c]), float(ths[n, c]), 0.5, 1.0, w)
        spikes += sum(ref[4])
        for got, want in zip(outs, ref[:4]):
            assert np.array_equal(got[n, c].numpy(), np.array(want, dtype=np.float32))
    assert spikes > 0
    # it is the resonator followed by the adaptive threshold driven by the imaginary trace
    re, im = O.res_fwd(xr, xi, torch.tensor(sin), torch.tensor(cos), rs, is_, w)
    th, ref = O.ath_fwd(im, refs, torch.tensor(rdl), ths, torch.tensor(tdl), 0.5, 1.0, w)
    for got, want in zip(outs, (re, im, th, ref)):
        assert torch.equal(got, want)


# ----------------------------------------------------------------------- RES
@pytest.mark.parametrize('thr', [None, 0.0, 1.5, 2.3])
def test_res_matches_scalar_spec(thr):
    rng = np.random.default_rng(31)
    T, w = 50, 64
    sin = [2103.0, 1.0, 3000.5, -2000.0]
    cos = [3273.0, 4095.0, 0.0, 2500.0]
    C = len(sin)
    xr = _rand_input(rng, (2, C, T))
    xi = _rand_input(rng, (2, C, T))
    rs = torch.tensor(rng.standard_normal((2, C)), dtype=torch.float32)
    is_ = torch.tensor(rng.standard_normal((2, C)), dtype=torch.float32)
    re, im = O.res_fwd(xr, xi, torch.tensor(sin), torch.tensor(cos), rs, is_, w, thr)
    for n, c in itertools.product(range(2), range(C)):
        r_ref, i_ref, _ = S.res(xr[n, c].tolist(), xi[n, c].tolist(), sin[c], cos[c],
                                float(rs[n, c]), float(is_[n, c]), w, thr)
        assert np.array_equal(re[n, c].numpy(), np.array(r_ref, dtype=np.float32))
        assert np.array_equal(im[n, c].numpy(), np.array(i_ref, dtype=np.float32))


def test_res_magnitude_and_phase():
    """Impulse response rotates by atan2(sin, cos) and shrinks by hypot/4096 per step
    (the reference's estimate, tests/.../dynamics/test_resonator.py:101-140)."""
    w = 1 << 12
    x = torch.zeros(1, 1, 40)
    x[..., 0] = 100.0
    s, c = 2103.0, 3273.0
    re, im = O.res_fwd(x, torch.zeros_like(x), torch.tensor([s]), torch.tensor([c]),
                       torch.tensor([0.0]), torch.tensor([0.0]), w)
    z = (re + 1j * im)[0, 0].numpy()
    ratio = z[1:] / z[:-1]
    assert np.allclose(np.abs(ratio), np.hypot(s, c) / 4096, rtol=1e-3)
    assert np.allclose(np.angle(ratio), np.arctan2(s, c), atol=1e-3)


def test_res_bwd_is_adjoint_of_float_rotation():
    rng = np.random.default_rng(33)
    N, C, T = 2, 3, 31
    f = lambda: torch.tensor(rng.standard_normal((N, C, T)), dtype=torch.float32)
    g_re, g_im, re, im = f(), f(), f(), f()
    sin = torch.tensor([2103.0, 500.0, 3000.0])
    cos = torch.tensor([3273.0, 3900.0, 100.0])
    gr, gi, gs, gc = O.res_bwd(g_re, g_im, re, im, sin, cos)
    sv = (sin.double() / 4096).requires_grad_()
    cv = (cos.double() / 4096).requires_grad_()
    xr = torch.zeros(N, C, T, dtype=torch.float64, requires_grad=True)
    xi = torch.zeros(N, C, T, dtype=torch.float64, requires_grad=True)
    a = torch.zeros(N, C, dtype=torch.float64)
    b = torch.zeros(N, C, dtype=torch.float64)
    outs_r, outs_i = [], []
    for t in range(T):
        a, b = cv * a - sv * b + xr[..., t], sv * a + cv * b + xi[..., t]
        outs_r.append(a)
        outs_i.append(b)
    (torch.stack(outs_r, -1) * g_re.double() + torch.stack(outs_i, -1) * g_im.double()).sum().backward()
    assert np.allclose(gr.numpy(), xr.grad.numpy(), rtol=1e-5, atol=1e-5)
    assert np.allclose(gi.numpy(), xi.grad.numpy(), rtol=1e-5, atol=1e-5)
    d = lambda v: v.double()
    ref_s = (-d(gr)[..., 1:] * d(im)[..., :-1] + d(gi)[..., 1:] * d(re)[..., :-1]).sum(dim=(0, 2))
    ref_c = (d(gr)[..., 1:] * d(re)[..., :-1] + d(gi)[..., 1:] * d(im)[..., :-1]).sum(dim=(0, 2))
    assert np.allclose(gs.numpy(), ref_s.numpy(), rtol=1e-5, atol=1e-5)
    assert np.allclose(gc.numpy(), ref_c.numpy(), rtol=1e-5, atol=1e-5)


def test_res_bwd_true_parameter_gradient():
    rng = np.random.default_rng(34)
    T = 20
    f = lambda: torch.tensor(rng.standard_normal((2, 1, T)), dtype=torch.float64)
    xr, xi, g_re, g_im = f(), f(), f(), f()
    sv = torch.tensor([0.4], dtype=torch.float64, requires_grad=True)
    cv = torch.tensor([0.7], dtype=torch.float64, requires_grad=True)
    a = torch.zeros(2, 1, dtype=torch.float64)
    b = torch.zeros(2, 1, dtype=torch.float64)
    rs, is_ = [], []
    for t in range(T):
        a, b = cv * a - sv * b + xr[..., t], sv * a + cv * b + xi[..., t]
        rs.append(a)
        is_.append(b)
    re, im = torch.stack(rs, -1), torch.stack(is_, -1)
    (re * g_re + im * g_im).sum().backward()
    _, _, gs, gc = O.res_bwd(g_re.float(), g_im.float(), re.detach().float(), im.detach().float(),
                             torch.tensor([0.4 * 4096]), torch.tensor([0.7 * 4096]))
    assert np.isclose(gs.item(), sv.grad.item(), rtol=1e-4)
    assert np.isclose(gc.item(), cv.grad.item(), rtol=1e-4)


def test_res_bwd_nan_guard():
    z = torch.zeros(1, 1, 4)
    bad = z.clone()
    bad[..., 2] = float('nan')
    with pytest.raises(Exception):
        O.res_bwd(bad, z, z, z, torch.tensor([1.0]), torch.tensor([1.0]))


# -------------------------------------------------------------------- spikes
def test_spike_closed_forms():
    rng = np.random.default_rng(40)
    v = torch.tensor(rng.standard_normal((2, 3, 50)) * 2, dtype=torch.float32)
    g = torch.tensor(rng.standard_normal((2, 3, 50)), dtype=torch.float32)
    th, tau, rho = 0.7, 1.3, 0.9
    assert np.array_equal(O.spike_fwd(v, th).numpy(), (v.numpy() >= np.float32(th)).astype(np.float32))
    d = v.double().numpy() - np.float32(th)
    ref = rho / (2 * tau) * np.exp(-np.abs(d) / tau) * g.double().numpy()
    assert np.allclose(O.spike_bwd(g, v, th, tau, rho).numpy(), ref, rtol=1e-5, atol=1e-7)
    ref = rho * np.exp(np.minimum(d, 0) / tau) * g.double().numpy()
    assert np.allclose(O.spike_bwd(g, v, th, tau, rho, graded=True).numpy(), ref, rtol=1e-5, atol=1e-7)
    # graded forward carries the voltage, tensor threshold is elementwise
    tht = torch.tensor(rng.standard_normal((2, 3, 50)), dtype=torch.float32)
    s = O.spike_fwd(v, tht, graded=True, scale=4)
    assert torch.equal(s, torch.where(v >= tht, v, torch.zeros_like(v)) / 4)


def test_cspike_closed_forms():
    rng = np.random.default_rng(41)
    f = lambda: torch.tensor(rng.standard_normal((2, 3, 40)) * 2, dtype=torch.float32)
    re, im, g = f(), f(), f()
    th, tau, rho = 0.4, 0.5, 10.0
    last = torch.tensor(rng.standard_normal((2, 3)), dtype=torch.float32)
    s = O.cspike_fwd(re, im, th, last).numpy()
    imn, ren = im.numpy(), re.numpy()
    for n, c, t in itertools.product(range(2), range(3), range(40)):
        prev = last[n, c].item() if t == 0 else imn[n, c, t - 1]
        assert s[n, c, t] == float(ren[n, c, t] >= np.float32(th) and prev < 0 and imn[n, c, t] >= 0)
    r, i = re.double().numpy(), im.double().numpy()
    d_re = np.exp(-np.abs(r - np.float32(th)) / tau) / (2 * tau)
    d_im = np.exp(-np.abs(i) / tau) / (2 * tau)
    H = 0.5 * (1 + np.sign(r - np.float32(th)) * (1 - 2 * tau * d_re))
    a, b = O.cspike_bwd(g, re, im, th, tau, rho)
    assert np.allclose(a.numpy(), g.numpy() * rho * d_re * d_im, rtol=1e-5, atol=1e-7)
    # H = (1 + sign * (1 - 2 tau d_re)) / 2 cancels in float32 where real < threshold:
    # its absolute error is one float32 ulp of 1, so the check is absolute here
    ref_b = g.numpy() * (-rho / tau) * np.sign(i) * d_im * H
    assert np.allclose(b.numpy(), ref_b, rtol=1e-5, atol=2e-6 * np.abs(g.numpy()).max() * rho / tau)


# --------------------------------------------------------------------- shift
def test_shift_matches_numpy_slicing():
    rng = np.random.default_rng(50)
    x = torch.tensor(rng.random((3, 7, 90)), dtype=torch.float32)
    xn = x.numpy()
    for k in (10, -10, 0, 89, 90, -95, 2.7, -2.7):
        ref = np.zeros_like(xn)
        kk = int(k)
        if kk == 0:
            ref = xn.copy()
        elif 0 < kk < 90:
            ref[..., kk:] = xn[..., :-kk]
        elif -90 < kk < 0:
            ref[..., :kk] = xn[..., -kk:]
        assert np.array_equal(O.shift(x, k).numpy(), ref), k
    lut = torch.arange(7, dtype=torch.float32) * 3.5 - 10
    out = O.shift(x, lut).numpy()
    for c in range(7):
        assert np.array_equal(out[:, c], O.shift(x[:, c:c + 1], int(lut[c].item())).numpy()[:, 0])
    # sampling time divides the shift (scalar form)
    assert torch.equal(O.shift(x, 6, sampling_time=2), O.shift(x, 3))
    with pytest.raises(Exception):
        O.shift(x, torch.arange(6, dtype=torch.float32))
    with pytest.raises(AssertionError):
        O.shift(torch.zeros(5), 1)
    # spatial tensors: one shift per (C,H,W) neuron
    x5 = torch.tensor(rng.random((2, 2, 3, 2, 30)), dtype=torch.float32)
    lut5 = torch.tensor(rng.integers(-5, 6, (2, 3, 2)), dtype=torch.float32)
    o5 = O.shift(x5, lut5)
    for c, h, w in itertools.product(range(2), range(3), range(2)):
        assert torch.equal(o5[:, c, h, w], O.shift(x5[:, c, h, w], int(lut5[c, h, w])))


# ---------------------------------------------------------------------- conv
def test_conv_corr_match_numpy_convolve():
    rng = np.random.default_rng(60)
    x = torch.tensor(rng.random((5, 4, 120)), dtype=torch.float32)
    f = torch.tensor(rng.random(17), dtype=torch.float32)
    y = O.conv_fwd(x, f, 0.5).numpy()
    z = O.conv_bwd(x, f, 0.5).numpy()
    for n, c in itertools.product(range(5), range(4)):
        row = x[n, c].double().numpy()
        assert np.allclose(y[n, c], 0.5 * np.convolve(row, f.double().numpy())[:120], rtol=1e-5, atol=1e-6)
        assert np.allclose(z[n, c], 0.5 * np.convolve(row[::-1], f.double().numpy())[:120][::-1],
                           rtol=1e-5, atol=1e-6)
    # adjointness <conv(x), g> == <x, corr(g)>
    g = torch.tensor(rng.random((5, 4, 120)), dtype=torch.float32)
    lhs = (O.conv_fwd(x, f).double() * g.double()).sum()
    rhs = (x.double() * O.conv_bwd(g, f).double()).sum()
    assert np.isclose(lhs.item(), rhs.item(), rtol=1e-5)


def test_delay_bwd():
    rng = np.random.default_rng(70)
    x = torch.tensor(rng.random((2, 3, 40)), dtype=torch.float32)
    d = torch.tensor([0.0, 3.2, 7.9])
    out = O.delay_fwd(x, d)
    for c, k in enumerate((0, 3, 7)):
        assert torch.equal(out[:, c, k:], x[:, c, :40 - k])
    g = torch.tensor(rng.standard_normal((2, 3, 40)), dtype=torch.float32)
    gi, gd = O.delay_bwd(g, out, d, grad_scale=2.0)
    for c, k in enumerate((0, 3, 7)):
        assert torch.equal(gi[:, c, :40 - k], g[:, c, k:])
    o = out.double().numpy()
    diff = np.zeros_like(o)
    diff[..., 0] = -o[..., 0]
    diff[..., 1:] = o[..., :-1] - o[..., 1:]
    assert np.allclose(gd.numpy(), 2.0 * (g.double().numpy() * diff).sum(axis=(0, 2)), rtol=1e-5, atol=1e-6)


# --------------------------------------------------------------------------------- sigma-delta
def test_delta_hand_sequences_and_reconstruction():
    z = torch.zeros(1, 1)
    x = torch.tensor([[[0.0, 0.4, 0.9, 1.0, 1.0, 0.2, -1.0]]])
    thr = torch.tensor([0.5])
    out, d_in, res, err = O.delta_fwd(x, thr, z, z, z)
    # changes: .4 (kept as residual), .5+.4=.9 (event), .1 (residual), 0+.1 (residual .1), -.8+.1=-.7 (event), -1.2 (event)
    assert np.allclose(out[0, 0].numpy(), [0, 0, 0.9, 0, 0, -0.7, -1.2], atol=1e-6)
    assert np.allclose(d_in[0, 0].numpy(), [0, 0.4, 0.9, 0.1, 0.1, -0.7, -1.2], atol=1e-6)
    assert abs(res.item()) < 1e-6
    # cumulative error: 0.2 stays below 0.5 (residual 0.2); the next change 0.2 + 0.2 brings the error to 0.6,
    # an event of 0.4 fires and the error restarts; the pattern repeats
    x = torch.tensor([[[0.2, 0.4, 0.6, 0.8]]])
    out, _, _, err = O.delta_fwd(x, thr, z, z, z, cum_error=True)
    assert np.allclose(out[0, 0].numpy(), [0, 0.4, 0, 0.4], atol=1e-6) and abs(err.item()) < 1e-6
    # without the cumulative error the same input never reaches the threshold in one step until the residual does
    out, _, _, _ = O.delta_fwd(x, thr, z, z, z, cum_error=False)
    assert np.allclose(out[0, 0].numpy(), [0, 0, 0.6, 0], atol=1e-6)
    # reconstruction: the decoder follows the signal within one threshold, exactly where an event fired
    rng = np.random.default_rng(80)
    x = torch.tensor(np.cumsum(rng.standard_normal((3, 5, 200)) * 0.3, axis=-1), dtype=torch.float32)
    zero = torch.zeros(3, 5)
    for cum in (False, True):
        out, _, res, _ = O.delta_fwd(x, thr, zero, zero, zero, cum)
        rec = O.sigma_fwd(out)
        assert float((x - rec).abs().max()) < (0.5 if not cum else 3.0) + 1e-4
        fired = out != 0
        assert fired.any()
        if not cum:
            assert float((x - rec)[fired].abs().max()) < 1e-4
            assert np.allclose(res.numpy(), (x - rec)[..., -1].numpy(), atol=1e-4)
    # carried state: splitting time gives the same events
    out, _, _, _ = O.delta_fwd(x, thr, zero, zero, zero)
    a, _, res_a, err_a = O.delta_fwd(x[..., :77], thr, zero, zero, zero)
    b, _, _, _ = O.delta_fwd(x[..., 77:], thr, x[..., 76], res_a, err_a)
    assert torch.equal(torch.cat([a, b], -1), out)
    # torch's CPU cumsum does not add strictly one float32 at a time, so the running sum is a float-mode
    # quantity (1e-5 relative); on event values that are multiples of 1/64 every order gives the same bits
    assert np.allclose(O.sigma_fwd(out).numpy(), np.cumsum(out.double().numpy(), axis=-1), rtol=1e-5, atol=1e-5)
    q = O.quantize_floor(out, 1 / 64)
    assert np.array_equal(O.sigma_fwd(q).numpy(), np.cumsum(q.double().numpy(), axis=-1).astype(np.float32))


def test_delta_bwd_closed_form():
    rng = np.random.default_rng(81)
    d = torch.tensor(rng.standard_normal((2, 3, 4, 30)), dtype=torch.float32)
    g = torch.tensor(rng.standard_normal((2, 3, 4, 30)), dtype=torch.float32)
    for thr in (torch.tensor([0.7]), torch.tensor([0.3, 0.7, 1.1]).reshape(3, 1)):
        g_in, g_thr = O.delta_bwd(g, d, thr, 0.8, 1.5)
        gn = g.double().numpy()
        ref_in = gn.copy()
        ref_in[..., :-1] -= gn[..., 1:]
        assert np.allclose(g_in.numpy(), ref_in, atol=1e-6)
        dn = d.double().numpy()
        th = thr.double().numpy().reshape(-1, 1, 1) if thr.numel() > 1 else thr.double().numpy()
        sub = np.abs(dn) - th
        term = np.where(sub > 0, -dn * 1.5 * np.exp(-np.abs(sub) / 0.8) / th, -np.sign(dn)) * gn
        want = term.sum() if thr.numel() == 1 else term.sum(axis=(0, 2, 3))
        assert np.allclose(g_thr.numpy().ravel(), np.ravel(want), rtol=1e-5, atol=1e-5)


def test_conv_synapse_is_the_defining_sum():
    """The convolution synapse (synapse/layer.py:297-323 in the reference, torch's conv3d with a (kh, kw, 1) kernel):
    out[n, co, ho, wo, t] = sum over ci, y, x of w[co, ci, y, x] * in[n, ci, ho * s + y * d - p, wo * s + x * d - p, t],
    written out as loops on small cases, strides, paddings, dilations and groups included.  A transposed kernel, a
    swapped stride / dilation or a wrong padding origin fails it."""
    gen = torch.Generator().manual_seed(5)
    for (ci, co, h, w, kh, kw, st, pd, dl, gr) in [(3, 4, 5, 6, 3, 3, (1, 1), (1, 1), (1, 1), 1),
                                                   (2, 4, 7, 5, 2, 3, (2, 1), (0, 2), (1, 2), 1),
                                                   (4, 6, 6, 6, 3, 2, (1, 2), (2, 0), (2, 1), 2)]:
        x = torch.randn(2, ci, h, w, 3, generator=gen)
        wt = torch.randn(co, ci // gr, kh, kw, 1, generator=gen)
        got = O.conv_synapse(x, wt, st, pd, dl, gr).double()
        ho = (h + 2 * pd[0] - dl[0] * (kh - 1) - 1) // st[0] + 1
        wo = (w + 2 * pd[1] - dl[1] * (kw - 1) - 1) // st[1] + 1
        assert got.shape == (2, co, ho, wo, 3)
        want = torch.zeros(2, co, ho, wo, 3, dtype=torch.float64)
        per_in, per_out = ci // gr, co // gr
        for o in range(co):
            g0 = (o // per_out) * per_in
            for c in range(per_in):
                for y in range(kh):
                    for xk in range(kw):
                        for a in range(ho):
                            for b in range(wo):
                                yy, xx = a * st[0] + y * dl[0] - pd[0], b * st[1] + xk * dl[1] - pd[1]
                                if 0 <= yy < h and 0 <= xx < w:
                                    want[:, o, a, b] += float(wt[o, c, y, xk, 0]) * x[:, g0 + c, yy, xx].double()
        assert float((got - want).abs().max()) < 1e-5
