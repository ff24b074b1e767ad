"""The oracle against the known-answer data the reference's own tests hold
(tests/lava/lib/dl/netx/test_blocks.py:180-332 in the reference tree), plus
mutations showing that each fixture is sensitive to the rule it pins."""
import numpy as np
import pytest
import torch

from oracle import slayer_oracle as O
from tests.golden import fixtures as G

W = G.W_SCALE
zero = torch.tensor([0.0])


def _mismatch(spikes, expected):
    s = spikes[0].numpy().astype(np.int64)[:, :expected.shape[1]]
    return int((s != expected).sum())


def _cuba(fx, cdecay=None, vdecay=None, thr=None, shift_fn=None):
    cdecay = fx['current_decay'] if cdecay is None else cdecay
    vdecay = fx['voltage_decay'] if vdecay is None else vdecay
    thr = fx['threshold'] if thr is None else thr
    cur = O.li_fwd(fx['x'], torch.tensor([cdecay]), zero, W)
    vol = O.li_fwd(cur, torch.tensor([vdecay]), zero, W, threshold=thr)
    return O.spike_fwd(vol, thr)


def test_dense_lif_fixture_exact():
    fx = G.dense_lif()
    assert fx['expected'].sum() == 1826
    assert _mismatch(_cuba(fx), fx['expected']) == 0


def test_dense_lif_fixture_is_sensitive():
    fx = G.dense_lif()
    # threshold without the epsilon (v >= 384 instead of v > 384), decay off by one
    assert _mismatch(_cuba(fx, thr=6 / 64), fx['expected']) > 0
    assert _mismatch(_cuba(fx, vdecay=414.0), fx['expected']) > 0
    assert _mismatch(_cuba(fx, vdecay=416.0), fx['expected']) > 0
    # floor shift instead of truncation toward zero
    saved = O.rs0
    try:
        O.rs0 = lambda x, bits=12: x >> bits
        assert _mismatch(_cuba(fx), fx['expected']) > 0
    finally:
        O.rs0 = saved


def _rf(fx, sin=None, cos=None):
    sin = fx['sin_decay'] if sin is None else sin
    cos = fx['cos_decay'] if cos is None else cos
    re, im = O.res_fwd(fx['xr'], fx['xi'], torch.tensor([sin]), torch.tensor([cos]), zero, zero, W)
    return O.cspike_fwd(re, im, fx['threshold'])


def test_complex_dense_rf_fixture_exact():
    fx = G.complex_dense_rf()
    assert (fx['sin_decay'], fx['cos_decay']) == (2103.0, 3273.0)
    assert fx['expected'].sum() > 40000
    assert _mismatch(_rf(fx), fx['expected']) == 0


def test_complex_dense_rf_fixture_is_sensitive():
    fx = G.complex_dense_rf()
    assert _mismatch(_rf(fx, sin=2104.0), fx['expected']) > 0
    assert _mismatch(_rf(fx, cos=3272.0), fx['expected']) > 0
    # swapped real / imaginary drive
    re, im = O.res_fwd(fx['xi'], fx['xr'], torch.tensor([2103.0]), torch.tensor([3273.0]), zero, zero, W)
    assert _mismatch(O.cspike_fwd(re, im, fx['threshold']), fx['expected']) > 0
    # wrong sign of the rotation
    re, im = O.res_fwd(fx['xr'], fx['xi'], torch.tensor([-2103.0]), torch.tensor([3273.0]), zero, zero, W)
    assert _mismatch(O.cspike_fwd(re, im, fx['threshold']), fx['expected']) > 0


def _rf_iz(fx, thr=None):
    thr = fx['threshold'] if thr is None else thr
    re, im = O.res_fwd(fx['x'], fx['x'], torch.tensor([fx['sin_decay']]), torch.tensor([fx['cos_decay']]),
                       zero, zero, W, threshold=thr)
    return (im >= thr).float(), re, im


def test_rf_iz_threshold_mode_fixture_exact():
    """Pins the threshold branch of the resonator (reset real to 0, imag to thr*w - 1)."""
    fx = G.complex_input_rf_iz()
    assert fx['expected'].sum() == 13548
    s, _, _ = _rf_iz(fx)
    assert _mismatch(s, fx['expected']) == 0


def test_rf_iz_fixture_is_sensitive():
    fx = G.complex_input_rf_iz()
    # no reset at all
    re, im = O.res_fwd(fx['x'], fx['x'], torch.tensor([fx['sin_decay']]), torch.tensor([fx['cos_decay']]),
                       zero, zero, W)
    assert _mismatch((im >= fx['threshold']).float(), fx['expected']) > 0
    # a different threshold (71 instead of 70.4 in scaled units)
    s, _, _ = _rf_iz(fx, thr=71.5 / W)
    assert _mismatch(s, fx['expected']) > 0


def test_li_reset_beyond_float32_integers_matches_reference_vectors():
    """States beyond 2**24 next to a threshold: vectors computed by the reference's CPU branch
    (tests/golden/make_reference_vectors.py)."""
    li, _ = G.reference_big_state_vectors()
    assert len(li) == 4
    zero = torch.tensor([0.0])
    for case in li:
        assert float(case['out'].abs().max()) * G.W_SCALE > 2 ** 24
        got = O.li_fwd(case['x'], zero, zero, G.W_SCALE, case['threshold'])
        assert torch.equal(got, case['out']), case['threshold']


def test_resonator_threshold_mode_beyond_float32_integers_matches_reference_vectors():
    _, res = G.reference_big_state_vectors()
    assert len(res) == 3
    zero = torch.tensor([0.0])
    for case in res:
        assert float(case['im'].abs().max()) * G.W_SCALE > 2 ** 24
        re, im = O.res_fwd(case['xr'], case['xi'], case['sin'], case['cos'], zero, zero, G.W_SCALE, case['threshold'])
        assert torch.equal(re, case['re']), case['threshold']
        assert torch.equal(im, case['im']), case['threshold']


def _neuron_case(name):
    return next(c for c in G.reference_neuron_vectors() if c['name'] == name)


def _per_channel(v):
    return v.round()              # the neurons hand the dynamics rounded decays (quantize)


@pytest.mark.parametrize('name', ['alif_shared', 'alif_graded_channel'])
def test_oracle_chain_equals_the_reference_alif_neuron(name):
    """First call (initial states) of the reference's alif.Neuron, from tests/golden/reference_neuron_vectors.npz:
    li_fwd -> li_fwd -> ath_fwd -> spike_fwd composed the way neuron/alif.py:499-525,557-591 does, plus the
    states it carries over."""
    c = _neuron_case(name)
    k, p, x = c['kwargs'], c['params'], c['inputs'][0]
    w = k.get('scale', 64)
    s = w * 64
    thr = int(k['threshold'] * w) / w
    step = int(k['threshold_step'] * w) / w
    zero = torch.tensor([0.0])
    cur = O.li_fwd(x, _per_channel(p['current_decay']), zero, s)
    vol = O.li_fwd(cur, _per_channel(p['voltage_decay']), zero, s)
    th, ref = O.ath_fwd(vol, zero, _per_channel(p['refractory_decay']), torch.tensor([thr]),
                        _per_channel(p['threshold_decay']), step, thr, s)
    spk = O.spike_fwd(vol, th + ref, graded=k.get('graded_spike', False), scale=1)
    assert torch.equal(spk, c['outputs'][0])
    st = c['states'][0]
    assert torch.equal(cur[..., -1], st['current_state']) and torch.equal(vol[..., -1], st['voltage_state'])
    last = spk[..., -1]
    assert torch.equal(O.ath_persistent_ref_state(ref[..., -1], last, th[..., -1]), st['refractory_state'])
    assert torch.equal(O.ath_persistent_th_state(th[..., -1], last, step), st['threshold_state'])


@pytest.mark.parametrize('name', ['adrf_shared', 'adrf_channel', 'adrf_iz_shared', 'adrf_iz_graded'])
def test_oracle_chain_equals_the_reference_adaptive_resonators(name):
    """First call of adrf.Neuron (res_fwd -> apth_fwd -> complex spike, neuron/adrf.py:583-660) and of
    adrf_iz.Neuron (adres_fwd -> spike, neuron/adrf_iz.py:574-645): pins apth_fwd and adres_fwd to outputs of the
    reference itself."""
    c = _neuron_case(name)
    k, p = c['kwargs'], c['params']
    xr, xi = c['inputs'][0]
    w = k.get('scale', 64)
    s = w * 64
    thr = int(k['threshold'] * w) / w
    step = int(k['threshold_step'] * w) / w
    zero = torch.tensor([0.0])
    sin, cos = _per_channel(p['sin_decay']), _per_channel(p['cos_decay'])
    d_th, d_ref = _per_channel(p['threshold_decay']), _per_channel(p['refractory_decay'])
    graded = k.get('graded_spike', False)
    st = c['states'][0]
    if c['module'] == 'adrf':
        re, im = O.res_fwd(xr, xi, sin, cos, zero, zero, s)
        th, ref = O.apth_fwd(re, im, zero, zero, d_ref, torch.tensor([thr]), d_th, step, thr, s)
        spk = O.cspike_fwd(re, im, th + ref, 0.0, graded=graded, scale=1)
    else:
        re, im, th, ref = O.adres_fwd(xr, xi, sin, cos, d_ref, d_th, zero, zero, zero, torch.tensor([thr]), step, thr, s)
        spk = O.spike_fwd(im, th + ref, graded=graded, scale=1)
    assert float((spk != 0).float().mean()) > 0.02
    assert torch.equal(spk, c['outputs'][0])
    assert torch.equal(re[..., -1], st['real_state']) and torch.equal(im[..., -1], st['imag_state'])


def test_oracle_chain_equals_the_reference_sigma_delta_neuron():
    """sigma_delta.Neuron (neuron/sigma_delta.py:171-219): running sum -> activation -> delta encoder, both
    calls (the second starts from the carried sums and residuals)."""
    c = _neuron_case('sigma_delta_relu')
    thr = c['params']['delta.threshold']
    pre_sigma = None
    pre = res = err = torch.zeros(c['inputs'][0].shape[:-1])
    for call in (0, 1):
        dend = O.sigma_fwd(c['inputs'][call], pre_sigma)
        act = torch.relu(dend)
        out, _, res, err = O.delta_fwd(act, thr, pre, res, err)
        out = O.quantize_floor(out, 1 / 4096)            # Delta.forward floors its events to the state grid (64 * 64)
        assert float((out != 0).float().mean()) > 0.05
        assert torch.equal(out, c['outputs'][call]), call
        pre_sigma, pre = dend[..., -1], act[..., -1]
        st = c['states'][call]
        assert torch.allclose(pre_sigma, st['sigma.pre_state'], rtol=1e-5, atol=1e-6)      # summation order
        assert torch.allclose(res, st['delta.residual_state'], rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize('name', ['delay_nct', 'delay_nchwt', 'delay_ts2'])
def test_oracle_delay_against_the_reference_delay_module(name):
    """tests/golden/reference_delay_vectors.npz: the reference's own axon.Delay (CPU branch).  Its per-neuron shift
    divides by the sampling time twice (utils/time/shift.py:82,56), so its result for a delay d is the oracle's (one
    division, like the CUDA kernel) for d / Ts; at Ts = 1 the two coincide."""
    c = G.reference_delay_vectors()[name]
    ts, _, grad_scale = (float(v) for v in c['cfg'])
    d = c['delay'] / ts
    if c['in'].dim() > 3:
        tile = list(c['in'].shape[1:-1])
        tile[0] = 1
        d = d.reshape((-1,) + (1,) * (len(tile) - 1)).repeat(tile)
    assert torch.equal(O.delay_fwd(c['in'], d, ts), c['out'])
    g_in, g_d = O.delay_bwd(c['grad_out'], c['out'], d, grad_scale, ts)
    assert torch.equal(g_in, c['grad_in'])
    if c['in'].dim() == 3:
        assert torch.allclose(g_d, c['grad_delay'], rtol=1e-5, atol=1e-5)
    # a wrong sign of the shift back, or a shift of the output instead of the gradient, fails
    assert not torch.equal(O.shift(c['grad_out'], d, ts), c['grad_in'])


@pytest.mark.parametrize('name', ['shift_ts2', 'shift_ts_half'])
def test_oracle_shift_against_the_reference_at_other_sampling_times(name):
    c = G.reference_delay_vectors()[name]
    ts = float(c['ts'])
    assert torch.equal(O.shift(c['in'], c['shift'] / ts, ts), c['out'])
    assert not torch.equal(O.shift(c['in'], c['shift'], ts), c['out'])     # one division is a different result
