"""The resonator-family and sigma-delta neuron modules (rf_iz, adrf, adrf_iz, sigma_delta) on the GPU:
each module against the CPU oracle's operator chain, and the reference tests' persistent-state
invariant (a run split in two with carried state equals the full run;
tests/lava/lib/dl/slayer/neuron/test_rf_iz.py, test_adrf.py, test_adrf_iz.py, test_sigma_delta.py)."""
import numpy as np
import pytest
import torch

from oracle import slayer_oracle as O
from tests.util import dev, sparse_input, assert_exact, assert_rel

pytestmark = pytest.mark.gpu


@pytest.fixture(scope='module')
def slayer():
    import lava_dl_amd.slayer as s
    return s


def _q(param):
    return param.detach().round().cpu()


def _inputs(seed, shape, amp=1.0):
    gen = torch.Generator().manual_seed(seed)
    return sparse_input(gen, shape, p=0.3, amp=amp), sparse_input(gen, shape, p=0.3, amp=amp), gen


def test_rf_iz_neuron_matches_oracle_chain(slayer):
    shape = (2, 10, 200)
    xr, xi, gen = _inputs(201, shape)
    n = slayer.neuron.rf_iz.Neuron(threshold=1.0, period=9, decay=0.05).to(dev())
    a, b = xr.to(dev()).requires_grad_(), xi.to(dev()).requires_grad_()
    re, im = n.dynamics((a, b))
    spk = n.spike(re, im)
    zero = torch.tensor([0.0])
    r_re, r_im = O.res_fwd(xr, xi, _q(n.sin_decay), _q(n.cos_decay), zero, zero, 4096, 1.0)
    r_spk = O.spike_fwd(r_im, 1.0)
    assert_exact(re, r_re, 'rf_iz real'); assert_exact(im, r_im, 'rf_iz imag'); assert_exact(spk, r_spk, 'rf_iz spikes')
    assert 0 < float(r_spk.mean()) < 1
    g = torch.randn(shape, generator=gen)
    spk.backward(g.to(dev()))
    g_im = O.spike_bwd(g, r_im, 1.0, 100.0, 0.1)
    g_a, g_b, _, _ = O.res_bwd(torch.zeros_like(g_im), g_im, r_re, r_im, _q(n.sin_decay), _q(n.cos_decay))
    assert_rel(a.grad, g_a, 'rf_iz grad real input'); assert_rel(b.grad, g_b, 'rf_iz grad imag input')


def test_adrf_neuron_matches_oracle_chain(slayer):
    shape = (2, 10, 200)
    xr, xi, gen = _inputs(202, shape, amp=2.0)
    n = slayer.neuron.adrf.Neuron(threshold=1.0, threshold_step=0.5, period=9, decay=0.05,
                                  threshold_decay=0.1, refractory_decay=0.2).to(dev())
    re, im, th, ref = n.dynamics((xr.to(dev()), xi.to(dev())))
    spk = n.spike(re, im, th, ref)
    zero, one = torch.tensor([0.0]), torch.tensor([1.0])
    r_re, r_im = O.res_fwd(xr, xi, _q(n.sin_decay), _q(n.cos_decay), zero, zero, 4096)
    r_th, r_ref = O.apth_fwd(r_re, r_im, zero, zero, _q(n.refractory_decay), one, _q(n.threshold_decay),
                             0.5, 1.0, 4096)
    r_spk = O.cspike_fwd(r_re, r_im, r_th + r_ref, 0.0)
    for got, want, name in ((re, r_re, 'real'), (im, r_im, 'imag'), (th, r_th, 'threshold'),
                            (ref, r_ref, 'refractory'), (spk, r_spk, 'spikes')):
        assert_exact(got, want, f'adrf {name}')
    assert float(r_spk.sum()) > 0 and float((r_th != 1.0).float().sum()) > 0


def test_adrf_iz_neuron_matches_oracle_chain(slayer):
    shape = (2, 10, 200)
    xr, xi, gen = _inputs(203, shape, amp=2.0)
    n = slayer.neuron.adrf_iz.Neuron(threshold=1.0, threshold_step=0.5, period=9, decay=0.05,
                                     threshold_decay=0.1, refractory_decay=0.2).to(dev())
    a, b = xr.to(dev()).requires_grad_(), xi.to(dev()).requires_grad_()
    spk = n((a, b))
    zero, one = torch.tensor([0.0]), torch.tensor([1.0])
    r_re, r_im, r_th, r_ref = O.adres_fwd(xr, xi, _q(n.sin_decay), _q(n.cos_decay), _q(n.refractory_decay),
                                          _q(n.threshold_decay), zero, zero, zero, one, 0.5, 1.0, 4096)
    r_spk = O.spike_fwd(r_im, r_th + r_ref)
    assert_exact(spk, r_spk, 'adrf_iz spikes')
    assert float(r_spk.sum()) > 0
    g = torch.randn(shape, generator=gen)
    spk.backward(g.to(dev()))
    g_im = O.spike_bwd(g, r_im, r_th + r_ref, 100.0, 0.1)
    g_a, g_b, _, _ = O.res_bwd(torch.zeros_like(g_im), g_im, r_re, r_im, _q(n.sin_decay), _q(n.cos_decay))
    assert_rel(a.grad, g_a, 'adrf_iz grad real input'); assert_rel(b.grad, g_b, 'adrf_iz grad imag input')


@pytest.mark.parametrize('kind', ['rf_iz', 'adrf', 'adrf_iz'])
@pytest.mark.parametrize('shared', [True, False])
def test_persistent_state_split_invariance(slayer, kind, shared):
    shape, k = (3, 8, 120), 47
    xr, xi, _ = _inputs(204, shape, amp=2.0)
    x = (xr.to(dev()), xi.to(dev()))
    rng = lambda a, b: [a, b] if not shared else a
    torch.manual_seed(7)

    def mk(persistent):
        if kind == 'rf_iz':
            return slayer.neuron.rf_iz.Neuron(1.0, rng(5, 20) if not shared else 11, rng(0.02, 0.1),
                                              shared_param=shared, persistent_state=persistent).to(dev())
        cls = getattr(slayer.neuron, kind).Neuron
        return cls(1.0, 0.5, rng(5, 20) if not shared else 11, rng(0.02, 0.1), rng(0.05, 0.2), rng(0.1, 0.3),
                   shared_param=shared, persistent_state=persistent).to(dev())

    def run(n, inp):
        traces = n.dynamics(inp)
        return tuple(traces) + (n.spike(*traces),)

    full_n, split_n = mk(False), mk(True)
    full = run(full_n, x)
    split_n._prepare(x[0])
    for pa, pb in zip(full_n.parameters(), split_n.parameters()):
        pb.data = pa.data.clone()
    a = run(split_n, tuple(t[..., :k] for t in x))
    b = run(split_n, tuple(t[..., k:] for t in x))
    assert float(full[-1].sum()) > 0, 'no spikes in the test workload'
    for i, (f, pa, pb) in enumerate(zip(full, a, b)):
        assert torch.equal(torch.cat([pa, pb], dim=-1), f), f'{kind} trace {i} differs after the split'


@pytest.mark.parametrize('cum_error', [False, True])
def test_sigma_delta_neuron_matches_oracle_chain_and_split(slayer, cum_error):
    gen = torch.Generator().manual_seed(205)
    shape, k = (2, 6, 5, 90), 31
    x = (torch.randn(shape, generator=gen) * (torch.rand(shape, generator=gen) < 0.4)).mul(64).round().div(64)
    n = slayer.neuron.sigma_delta.Neuron(0.25, torch.relu, cum_error=cum_error).to(dev())
    out = n(x.to(dev()))
    zero = torch.zeros(shape[:-1])
    act = torch.relu(O.sigma_fwd(x))
    ev, _, _, _ = O.delta_fwd(act, torch.tensor([0.25]), zero, zero, zero, cum_error)
    want = O.quantize_floor(ev, 1 / 4096)
    assert_exact(out, want, 'sigma_delta events')
    assert 0 < float((want != 0).float().mean()) < 1
    m = slayer.neuron.sigma_delta.Neuron(0.25, torch.relu, cum_error=cum_error, persistent_state=True).to(dev())
    parts = torch.cat([m(x[..., :k].to(dev())), m(x[..., k:].to(dev()))], dim=-1)
    assert torch.equal(parts, out), 'sigma_delta output differs after the split'


def _reference_neuron_cases():
    from tests.golden import fixtures as G
    return G.reference_neuron_vectors()


@pytest.mark.parametrize('case', _reference_neuron_cases(), ids=lambda c: c['name'])
def test_neurons_against_vectors_of_the_reference_classes(slayer, case):
    """alif / adrf / adrf_iz / sigma_delta neurons against outputs of the reference's own classes
    (tests/golden/make_reference_neuron_vectors.py): same constructor arguments and parameters, two consecutive
    calls with persistent state; spikes (graded values included) and every carried state must be equal."""
    module = getattr(slayer.neuron, case['module'])
    kwargs = dict(case['kwargs'], persistent_state=True)
    if 'activation' in kwargs:
        kwargs['activation'] = {'relu': torch.relu}[kwargs['activation']]
    neuron = module.Neuron(**kwargs).to(dev())
    first = case['inputs'][0]
    gpu = (lambda x: tuple(t.to(dev()) for t in x) if isinstance(x, tuple) else x.to(dev()))
    if hasattr(neuron, '_prepare'):
        neuron._prepare(first[0].to(dev()) if isinstance(first, tuple) else first.to(dev()))
    with torch.no_grad():
        for pname, value in case['params'].items():
            owner = neuron
            *path, leaf = pname.split('.')
            for part in path:
                owner = getattr(owner, part)
            getattr(owner, leaf).data = value.to(dev()).reshape(getattr(owner, leaf).shape
                                                                if getattr(owner, leaf).numel() == value.numel()
                                                                else value.shape)
        for call in (0, 1):
            out = neuron(gpu(case['inputs'][call]))
            want = case['outputs'][call]
            assert float((want != 0).float().mean()) > 0.02
            assert_exact(out, want, f"{case['name']} output of call {call}")
            for sname, value in case['states'][call].items():
                owner = neuron
                *path, leaf = sname.split('.')
                for part in path:
                    owner = getattr(owner, part)
                if case['module'] == 'sigma_delta':
                    # the running sum of arbitrary floats: torch.cumsum groups the additions differently on every
                    # backend (sequential here), the last bits of the carried sums may differ
                    assert_rel(getattr(owner, leaf), value, f"{case['name']} {sname} after call {call}", rel=1e-5)
                else:
                    assert_exact(getattr(owner, leaf), value, f"{case['name']} {sname} after call {call}")


def _with_parameters(neuron, case, first):
    if hasattr(neuron, '_prepare'):
        neuron._prepare(first[0] if isinstance(first, tuple) else first)
    with torch.no_grad():
        for pname, value in case['params'].items():
            owner = neuron
            *path, leaf = pname.split('.')
            for part in path:
                owner = getattr(owner, part)
            prm = getattr(owner, leaf)
            prm.data = value.to(dev()).reshape(prm.shape if prm.numel() == value.numel() else value.shape)
    return neuron


@pytest.mark.parametrize('case', _reference_neuron_cases(), ids=lambda c: c['name'])
def test_neuron_gradients_against_vectors_of_the_reference_classes(slayer, case):
    """Input gradients of the same neurons (surrogate constants, which tensors the gradient flows through):
    d sum(output * g) / d input from the reference's own autograd, within 1e-5 relative."""
    module = getattr(slayer.neuron, case['module'])
    kwargs = dict(case['kwargs'])
    if 'activation' in kwargs:
        kwargs['activation'] = {'relu': torch.relu}[kwargs['activation']]
    neuron = module.Neuron(**kwargs).to(dev())
    first = case['inputs'][0]
    leaves = [t.to(dev()).requires_grad_() for t in (first if isinstance(first, tuple) else (first,))]
    _with_parameters(neuron, case, tuple(leaves) if len(leaves) == 2 else leaves[0])
    out = neuron(tuple(leaves) if len(leaves) == 2 else leaves[0])
    assert_exact(out, case['outputs'][0], f"{case['name']} output")
    out.backward(case['grad_out'].to(dev()))
    for i, want in enumerate(case['grad_in']):
        assert float(want.abs().max()) > 0
        assert_rel(leaves[i].grad, want, f"{case['name']} gradient of input {i}")
