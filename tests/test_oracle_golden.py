"""The oracle against the known-answer data the reference's own tests hold
(tests/lava/lib/dl/netx/test_blocks.py:180-332 in the reference tree), plus
mutations showing that each fixture is sensitive to the rule it pins."""
import numpy as np
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
