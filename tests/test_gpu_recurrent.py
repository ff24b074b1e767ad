"""Recurrent CUBA / ALIF layers, binary and graded spikes: the one-launch time loop against the CPU oracle
(bit-exact spikes, voltages and carried states with quantised weights), against the loops of one-step neuron
calls (the reference's own check, tests/lava/lib/dl/slayer/utils/test_recurrent.py:101-190), and the fallback
for layers the kernel does not cover."""
import pytest
import torch

from oracle import slayer_oracle as O
from tests.util import dev, assert_exact, assert_rel

pytestmark = pytest.mark.gpu


@pytest.fixture(scope='module')
def slayer():
    import lava_dl_amd.slayer as s
    return s


@pytest.fixture(autouse=True)
def one_launch(slayer, monkeypatch):
    """The tests of this file are about the one-launch kernels: widths that would take a launch per step
    (tests/test_gpu_recurrent_steps.py) stay on them."""
    monkeypatch.setattr(slayer.utils.recurrent, 'STEPS_FROM', 10 ** 9)


class _Dense(torch.nn.Module):
    """Stand-in for the dense synapse the layer is used with: weight [C_out, C_in, 1, 1, 1], optional pre-hook."""

    def __init__(self, n, gen):
        super().__init__()
        self.weight = torch.nn.Parameter((torch.randn(n, n, 1, 1, 1, generator=gen) * 0.6))
        self.pre_hook_fx = None

    def forward(self, x):                      # x: [N, C, 1]
        w = self.weight.reshape(self.weight.shape[:2])
        if self.pre_hook_fx is not None:
            w = self.pre_hook_fx(w)
        return torch.matmul(w, x)


def _sparse_weights(syn, gen, per_row=4):
    """A few weights of +-1/32 or +-2/32 per neuron.  Graded spikes feed voltages back: with current and voltage
    gains of 1 / decay each, the loop gain stays below one only for weights this small."""
    c = syn.weight.shape[0]
    w = torch.zeros(c, c)
    for row in range(c):
        cols = torch.randperm(c, generator=gen)[:per_row]
        w[row, cols] = (torch.randint(1, 3, (len(cols),), generator=gen) *
                        (2 * torch.randint(0, 2, (len(cols),), generator=gen) - 1)).float() / 32
    with torch.no_grad():
        syn.weight.copy_(w.reshape(syn.weight.shape))


def _neuron(slayer, **kw):
    args = dict(threshold=1.25, current_decay=0.25, voltage_decay=0.25, persistent_state=True)
    args.update(kw)
    return slayer.neuron.cuba.Neuron(**args).to(dev())


@pytest.mark.parametrize('n,c,t,shared', [(2, 10, 128, True), (3, 70, 100, False), (4, 300, 37, True), (1, 64, 4, True)])
def test_fused_loop_matches_the_oracle(slayer, n, c, t, shared):
    gen = torch.Generator().manual_seed(1000 * n + c + t)
    z = torch.randn(n, c, t, generator=gen)
    neuron = _neuron(slayer, shared_param=shared, current_decay=[0.2, 0.4] if not shared else 0.25,
                     voltage_decay=[0.1, 0.3] if not shared else 0.25)
    syn = _Dense(c, gen).to(dev())
    syn.pre_hook_fx = neuron.quantize_8bit
    zg = z.to(dev()).requires_grad_()
    out = slayer.utils.recurrent.custom_recurrent(zg, neuron, syn)
    rec = neuron.quantize_8bit(syn.weight.detach().reshape(c, c)).cpu()
    d_i, d_v = neuron.current_decay.detach().round().cpu(), neuron.voltage_decay.detach().round().cpu()
    thr = neuron.threshold + neuron.threshold_eps
    zero = torch.tensor([0.0])
    r_spk, r_vol, r_cs, r_vs = O.recurrent_cuba_fwd(z, rec, d_i, d_v, zero, zero, 4096, thr)
    assert 0.01 < float(r_spk.mean()) < 0.9, 'the case must spike, and the feedback must matter'
    assert_exact(out, r_spk, 'recurrent spikes')
    assert_exact(neuron.current_state, r_cs, 'carried current')
    assert_exact(neuron.voltage_state, r_vs, 'carried voltage')
    g = torch.rand(n, c, t, generator=gen)
    out.backward(g.to(dev()))
    r_gz, r_gw = O.recurrent_cuba_bwd(g, r_spk, r_vol, rec, thr, neuron.tau_rho * 100, neuron.scale_rho * 0.1)
    assert_rel(zg.grad, r_gz, 'recurrent grad z')
    assert_rel(syn.weight.grad.reshape(c, c), r_gw, 'recurrent grad weight')
    # a second call continues from the carried state
    out2 = slayer.utils.recurrent.custom_recurrent(z.to(dev()), neuron, syn)
    r_spk2, _, _, _ = O.recurrent_cuba_fwd(z, rec, d_i, d_v, r_cs, r_vs, 4096, thr)
    assert_exact(out2, r_spk2, 'recurrent spikes, second call')


def test_fused_loop_matches_the_loops_of_one_step_calls(slayer):
    gen = torch.Generator().manual_seed(298101)
    n, c, t = 2, 10, 128
    z = torch.randn(n, c, t, generator=gen).to(dev())
    R = slayer.utils.recurrent
    neurons = [_neuron(slayer, requires_grad=True) for _ in range(4)]
    syns = [_Dense(c, torch.Generator().manual_seed(5)).to(dev()) for _ in range(4)]
    for s, nrn in zip(syns, neurons):
        s.pre_hook_fx = nrn.quantize_8bit
    outs = [R.custom_recurrent(z, neurons[0], syns[0]),                                  # fused
            R.custom_recurrent_ground_truth_1(z, neurons[1], syns[1]),
            R.custom_recurrent_ground_truth_2(z, neurons[2], syns[2]),
            R.CustomRecurrent.apply(z, neurons[3], R._recurrent_matrix(syns[3]))]         # generic loop
    assert float(outs[0].detach().sum()) > 0
    for i in (1, 2, 3):
        assert torch.equal(outs[0], outs[i].detach()), f'forward differs from loop {i}'
    g = torch.rand(n, c, t, generator=gen).to(dev())
    for o in outs:
        torch.autograd.backward(o, g)
    for i in (1, 2, 3):
        assert_rel(syns[0].weight.grad.cpu(), syns[i].weight.grad.cpu(), f'weight gradient vs loop {i}')


def _alif(slayer, **kw):
    args = dict(threshold=1.0, threshold_step=0.5, current_decay=0.25, voltage_decay=0.1, threshold_decay=0.1,
                refractory_decay=0.2, persistent_state=True)
    args.update(kw)
    return slayer.neuron.alif.Neuron(**args).to(dev())


@pytest.mark.parametrize('n,c,t', [(2, 10, 128), (3, 70, 101), (2, 300, 36), (1, 1024, 8)])
@pytest.mark.parametrize('graded', [False, True])
def test_fused_alif_loop_matches_the_oracle(slayer, n, c, t, graded):
    gen = torch.Generator().manual_seed(77 * n + c + t + graded)
    z = torch.randn(n, c, t, generator=gen) * 2
    neuron = _alif(slayer, graded_spike=graded, **(dict(current_decay=0.5, voltage_decay=0.5) if graded else {}))
    syn = _Dense(c, gen).to(dev())
    if graded:
        _sparse_weights(syn, gen)
    else:
        with torch.no_grad():
            syn.weight.mul_(min(1.0, 6.0 / c ** 0.5))        # keep the feedback of the wide layers moderate
    syn.pre_hook_fx = neuron.quantize_8bit
    zg = z.to(dev()).requires_grad_()
    out = slayer.utils.recurrent.custom_recurrent(zg, neuron, syn)
    rec = neuron.quantize_8bit(syn.weight.detach().reshape(c, c)).cpu()
    names = ('current', 'voltage', 'threshold', 'refractory')
    decays = [getattr(neuron, f'{k}_decay').detach().round().cpu() for k in names]
    states = [torch.tensor([0.0]), torch.tensor([0.0]), torch.tensor([neuron.threshold]), torch.tensor([0.0])]
    r_spk, r_vol, r_theta, r_last = O.recurrent_alif_fwd(z, rec, decays, states, neuron.threshold_step,
                                                         neuron.threshold, 4096, graded=graded)
    assert 0.01 < float((r_spk != 0).float().mean()) < 0.9, 'the case must spike, and the feedback must matter'
    assert not torch.equal(r_spk, O.recurrent_alif_fwd(z, torch.zeros_like(rec), decays, states, neuron.threshold_step,
                                                       neuron.threshold, 4096, graded=graded)[0])
    assert_exact(out, r_spk, 'recurrent spikes')
    for k, want in zip(names, r_last):
        assert_exact(getattr(neuron, f'{k}_state'), want, f'carried {k}')
    g = torch.rand(n, c, t, generator=gen)
    out.backward(g.to(dev()))
    r_gz, r_gw = O.recurrent_cuba_bwd(g, r_spk, r_vol, rec, r_theta, neuron.tau_rho * 100, neuron.scale_rho * 0.1,
                                      graded=graded)
    assert_rel(zg.grad, r_gz, 'recurrent grad z')
    assert_rel(syn.weight.grad.reshape(c, c), r_gw, 'recurrent grad weight')
    # a second call continues from the carried state
    out2 = slayer.utils.recurrent.custom_recurrent(z.to(dev()), neuron, syn)
    r_spk2 = O.recurrent_alif_fwd(z, rec, decays, r_last, neuron.threshold_step, neuron.threshold, 4096,
                                  graded=graded)[0]
    assert_exact(out2, r_spk2, 'recurrent spikes, second call')


@pytest.mark.parametrize('n,c,t', [(2, 10, 128), (3, 70, 101), (2, 300, 36)])
def test_fused_cuba_loop_with_graded_spikes_matches_the_oracle(slayer, n, c, t):
    gen = torch.Generator().manual_seed(31 * n + c + t)
    z = torch.randn(n, c, t, generator=gen)
    neuron = _neuron(slayer, graded_spike=True)
    syn = _Dense(c, gen).to(dev())
    _sparse_weights(syn, gen)
    syn.pre_hook_fx = neuron.quantize_8bit
    zg = z.to(dev()).requires_grad_()
    out = slayer.utils.recurrent.custom_recurrent(zg, neuron, syn)
    rec = neuron.quantize_8bit(syn.weight.detach().reshape(c, c)).cpu()
    d_i, d_v = neuron.current_decay.detach().round().cpu(), neuron.voltage_decay.detach().round().cpu()
    thr = neuron.threshold + neuron.threshold_eps
    zero = torch.tensor([0.0])
    r_spk, r_vol, r_cs, r_vs = O.recurrent_cuba_fwd(z, rec, d_i, d_v, zero, zero, 4096, thr, graded=True)
    assert 0.01 < float((r_spk != 0).float().mean()) < 0.9
    assert float(r_spk.max()) > 1.3, 'graded spikes carry the voltage'
    assert_exact(out, r_spk, 'graded recurrent spikes')
    assert_exact(neuron.current_state, r_cs, 'carried current')
    assert_exact(neuron.voltage_state, r_vs, 'carried voltage')
    g = torch.rand(n, c, t, generator=gen)
    out.backward(g.to(dev()))
    r_gz, r_gw = O.recurrent_cuba_bwd(g, r_spk, r_vol, rec, thr, neuron.tau_rho * 100, neuron.scale_rho * 0.1,
                                      graded=True)
    assert_rel(zg.grad, r_gz, 'recurrent grad z')
    assert_rel(syn.weight.grad.reshape(c, c), r_gw, 'recurrent grad weight')


@pytest.mark.parametrize('kind,graded', [('alif', False), ('alif', True), ('cuba', True)])
def test_fused_loop_of_other_neurons_matches_the_loops_of_one_step_calls(slayer, kind, graded):
    gen = torch.Generator().manual_seed(4410 + graded)
    n, c, t = 2, 24, 90
    z = (torch.randn(n, c, t, generator=gen) * 1.5).to(dev())
    R = slayer.utils.recurrent
    mk = (lambda: _alif(slayer, graded_spike=graded, requires_grad=True, current_decay=0.5, voltage_decay=0.5)) \
        if kind == 'alif' else (lambda: _neuron(slayer, graded_spike=graded, requires_grad=True))
    neurons = [mk() for _ in range(3)]
    syns = [_Dense(c, torch.Generator().manual_seed(5)).to(dev()) for _ in range(3)]
    for s, nrn in zip(syns, neurons):
        s.pre_hook_fx = nrn.quantize_8bit
        if graded:
            _sparse_weights(s, torch.Generator().manual_seed(5))
    zs = [z.clone().requires_grad_() for _ in range(3)]
    outs = [R.custom_recurrent(zs[0], neurons[0], syns[0]),                                  # fused
            R.custom_recurrent_ground_truth_2(zs[1], neurons[1], syns[1]),
            R.CustomRecurrent.apply(zs[2], neurons[2], R._recurrent_matrix(syns[2]))]         # generic loop
    assert float((outs[0].detach() != 0).float().mean()) > 0.01
    for i in (1, 2):
        assert torch.equal(outs[0], outs[i].detach()), f'forward differs from loop {i}'
    g = torch.rand(n, c, t, generator=gen).to(dev())
    for o in outs:
        torch.autograd.backward(o, g)
    # the generic loop differentiates like the fused one (carried state = constant); autograd through the plain
    # loop also follows the carried states, so only the former is compared
    assert_rel(zs[0].grad.cpu(), zs[2].grad.cpu(), 'input gradient vs generic loop')
    assert_rel(syns[0].weight.grad.cpu(), syns[2].weight.grad.cpu(), 'weight gradient vs generic loop')
    for k in ('current', 'voltage') + (('threshold', 'refractory') if kind == 'alif' else ()):
        assert torch.equal(getattr(neurons[0], f'{k}_state'), getattr(neurons[2], f'{k}_state').reshape(n, c)), k


def test_layers_the_kernel_does_not_cover_take_the_generic_loop(slayer):
    gen = torch.Generator().manual_seed(7)
    n, c, t = 2, 12, 40
    z = torch.randn(n, c, t, generator=gen).mul(2).to(dev()).requires_grad_()
    R = slayer.utils.recurrent
    mk = lambda: _alif(slayer, dropout=slayer.neuron.Dropout(p=0.0))
    a, b = mk(), mk()
    assert not R._fusable(z, a) and R._fusable(z, _alif(slayer)) and not R._fusable(z, _alif(slayer, persistent_state=False))
    syn_a, syn_b = (_Dense(c, torch.Generator().manual_seed(3)).to(dev()) for _ in range(2))
    out = R.custom_recurrent(z, a, syn_a)
    ref = R.custom_recurrent_ground_truth_2(z.detach(), b, syn_b)
    assert torch.equal(out, ref.detach()) and float(out.detach().sum()) > 0
    out.sum().backward()
    assert torch.isfinite(z.grad).all() and syn_a.weight.grad is not None
