"""The axonal delay module and the per-neuron shift against vectors of the reference's own CPU branch
(tests/golden/make_reference_delay_vectors.py; axon/delay.py:132-221, utils/time/shift.py:46-143), through the
separate operators and folded into the fused CUBA kernel's spike store.

Sampling times other than 1: the reference's CPU branch divides a per-neuron shift by the sampling time twice
(utils/time/shift.py:82 and :56), its CUDA kernel once (utils/time/shift.cu:68).  This package divides once, like
the kernel it replaces; the vectors show the relation exactly: the reference's result for a shift d is this
package's result for d / Ts."""
import pytest
import torch

from oracle import slayer_oracle as O
from tests.golden import fixtures as G
from tests.util import dev, assert_exact, assert_rel

pytestmark = pytest.mark.gpu

CASES = G.reference_delay_vectors()


@pytest.fixture(scope='module')
def slayer():
    import lava_dl_amd.slayer as s
    return s


@pytest.mark.parametrize('name', ['delay_nct', 'delay_nchwt', 'delay_ts2'])
def test_delay_module_against_the_reference(slayer, name):
    c = CASES[name]
    ts, max_delay, grad_scale = (float(v) for v in c['cfg'])
    ts = int(ts) if ts == int(ts) else ts
    mod = slayer.axon.Delay(sampling_time=ts, max_delay=max_delay, grad_scale=grad_scale).to(dev())
    # the reference moved every row by trunc((d / Ts) / Ts) steps: for this package that is the delay d / Ts
    mod.delay.data = (c['delay'] / ts).to(dev())
    mod.init = True
    x = c['in'].to(dev()).requires_grad_()
    y = mod(x)
    assert_exact(y, c['out'], 'delayed output')
    assert float((c['out'] != c['in']).float().mean()) > 0.2
    y.backward(c['grad_out'].to(dev()))
    assert_exact(x.grad, c['grad_in'], 'gradient of the input')
    assert_rel(mod.delay.grad, c['grad_delay'], 'gradient of the delays', rel=1e-5)
    # the oracle agrees with the reference too
    r_out = O.delay_fwd(c['in'], _per_neuron(c['delay'] / ts, c['in']), ts)
    assert torch.equal(r_out, c['out'])
    r_gin, r_gd = O.delay_bwd(c['grad_out'], c['out'], _per_neuron(c['delay'] / ts, c['in']), grad_scale, ts)
    assert torch.equal(r_gin, c['grad_in'])
    want = c['grad_delay'] if c['in'].dim() == 3 else None
    if want is not None:
        assert_rel(r_gd, want, 'oracle gradient of the delays', rel=1e-5)


def _per_neuron(delay, like):
    if like.dim() == 3:
        return delay
    tile = list(like.shape[1:-1])
    tile[0] = 1
    return delay.reshape((-1,) + (1,) * (len(tile) - 1)).repeat(tile)


@pytest.mark.parametrize('name', ['shift_ts2', 'shift_ts_half'])
def test_per_neuron_shift_at_other_sampling_times(slayer, name):
    c = CASES[name]
    ts = float(c['ts'])
    got = slayer.utils.time.shift(c['in'].to(dev()), (c['shift'] / ts).to(dev()), ts)
    assert_exact(got, c['out'], 'shift with the reference\'s double division expressed as d / Ts')
    assert torch.equal(O.shift(c['in'], c['shift'] / ts, ts), c['out'])
    # and the rule this package documents: one division, truncation toward zero
    k = (c['shift'].flatten() / ts).to(torch.int32)
    once = slayer.utils.time.shift(c['in'].to(dev()), c['shift'].to(dev()), ts).cpu()
    rows = c['in'].reshape(c['in'].shape[0], -1, c['in'].shape[-1])
    T = rows.shape[-1]
    for r in range(rows.shape[1]):
        kr = int(k[r])
        want = torch.zeros_like(rows[:, r])
        if abs(kr) < T:
            if kr >= 0:
                want[:, kr:] = rows[:, r, :T - kr]
            else:
                want[:, :T + kr] = rows[:, r, -kr:]
        assert torch.equal(once.reshape(rows.shape)[:, r], want), f'row {r}: shift {kr}'


@pytest.mark.parametrize('name', ['delay_nct', 'delay_nchwt'])
def test_folded_delay_reproduces_the_reference_delay_module(slayer, name):
    """The fused CUBA kernel storing its spikes through the same delays: equal to the reference module applied to
    the undelayed spikes (forward), and the same delay gradient when the same gradient arrives."""
    c = CASES[name]
    ts, max_delay, grad_scale = (float(v) for v in c['cfg'])
    D = slayer.neuron.dynamics
    x = c['in'].to(dev())
    to = lambda t: t.to(dev())
    zero, di, dv = torch.zeros(1, device=dev()), torch.tensor([1024.0], device=dev()), torch.tensor([128.0], device=dev())
    plain = D.cuba_fused.spikes(x * 3, di, dv, zero, zero, 64, 0.5)[2]
    delay = _per_neuron(c['delay'], c['in']).to(dev()).requires_grad_()
    folded = D.delays.Delays(output_delay=delay, sampling_time=1, grad_scale=grad_scale)
    xg = (x * 3).requires_grad_()
    _, _, spk, _ = D.cuba_fused.dynamics(xg, di, dv, zero, zero, 64, 0.5, 1.0, 1.0, False, 1, keep_current=False,
                                         delays=folded)
    want = O.delay_fwd(plain.cpu(), _per_neuron(c['delay'], c['in']), 1)
    assert_exact(spk, want, 'spikes stored through the delays')
    assert float(plain.sum()) > 10
    spk.backward(to(c['grad_out']))
    _, r_gd = O.delay_bwd(c['grad_out'], want, _per_neuron(c['delay'], c['in']), grad_scale, 1)
    assert_rel(delay.grad.reshape(r_gd.shape), r_gd, 'delay gradient of the folded form')
