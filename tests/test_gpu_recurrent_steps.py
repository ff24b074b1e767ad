"""Recurrent CUBA / ALIF layers through the launch-per-step kernels (layers wider than one workgroup per sample
holds): the checks of the one-launch kernels repeated on this path (CPU oracle bit for bit with quantised weights,
the loops of one-step calls), the two paths against each other, and wide layers at their natural size."""
import pytest
import torch

from oracle import slayer_oracle as O
from tests import test_gpu_recurrent as base
from tests.util import dev, assert_exact, assert_rel

pytestmark = pytest.mark.gpu


@pytest.fixture(scope='module')
def slayer():
    import lava_dl_amd.slayer as s
    return s


@pytest.fixture()
def by_steps(slayer, monkeypatch):
    """Every layer whose width is a multiple of 4 takes the launch-per-step kernels; counts their calls."""
    R = slayer.utils.recurrent
    calls = []
    plain = R._steps_workspace

    def counted(*a):
        calls.append(a)
        return plain(*a)
    monkeypatch.setattr(R, 'STEPS_FROM', 0)
    monkeypatch.setattr(R, '_steps_workspace', counted)
    yield calls
    assert calls, 'the launch-per-step path was not taken'


# batch sizes on either side of 16, 32 and 64 samples (one, two, four sample tiles, two workgroups along the batch),
# widths that are not whole tiles of 16 neurons
@pytest.mark.parametrize('n,c,t,shared', [(2, 12, 128, True), (3, 68, 100, False), (4, 300, 37, True), (1, 64, 4, True),
                                          (17, 36, 21, True), (40, 20, 9, False), (70, 16, 6, True), (3, 516, 1, True)])
def test_cuba_layer_by_steps_matches_the_oracle(slayer, by_steps, n, c, t, shared):
    base.test_fused_loop_matches_the_oracle(slayer, n, c, t, shared)


@pytest.mark.parametrize('n,c,t', [(2, 12, 128), (3, 68, 101), (2, 300, 36), (33, 20, 17)])
@pytest.mark.parametrize('graded', [False, True])
def test_alif_layer_by_steps_matches_the_oracle(slayer, by_steps, n, c, t, graded):
    base.test_fused_alif_loop_matches_the_oracle(slayer, n, c, t, graded)


@pytest.mark.parametrize('n,c,t', [(2, 12, 128), (3, 68, 101), (2, 300, 36)])
def test_graded_cuba_layer_by_steps_matches_the_oracle(slayer, by_steps, n, c, t):
    base.test_fused_cuba_loop_with_graded_spikes_matches_the_oracle(slayer, n, c, t)


@pytest.mark.parametrize('kind,graded', [('alif', False), ('alif', True), ('cuba', True)])
def test_layer_by_steps_matches_the_loops_of_one_step_calls(slayer, by_steps, kind, graded):
    base.test_fused_loop_of_other_neurons_matches_the_loops_of_one_step_calls(slayer, kind, graded)


@pytest.mark.parametrize('kind', ['cuba', 'alif'])
def test_the_two_kernel_paths_agree(slayer, monkeypatch, kind):
    """One layer through the one-launch kernels and through the launch-per-step kernels: the same spikes and carried
    states bit for bit (quantised weights), the same gradients to summation order."""
    R = slayer.utils.recurrent
    gen = torch.Generator().manual_seed(90210)
    n, c, t = 5, 512, 64
    z = (torch.randn(n, c, t, generator=gen) * 1.5).to(dev())
    g = torch.rand(n, c, t, generator=gen).to(dev())
    results = []
    for first in (10 ** 9, 0):
        monkeypatch.setattr(R, 'STEPS_FROM', first)
        neuron = base._alif(slayer) if kind == 'alif' else base._neuron(slayer)
        syn = base._Dense(c, torch.Generator().manual_seed(5)).to(dev())
        with torch.no_grad():
            syn.weight.mul_(6.0 / c ** 0.5)
        syn.pre_hook_fx = neuron.quantize_8bit
        zg = z.clone().requires_grad_()
        out = R.custom_recurrent(zg, neuron, syn)
        out.backward(g)
        results.append((out.detach(), zg.grad, syn.weight.grad, neuron.current_state, neuron.voltage_state))
    a, b = results
    assert 0.01 < float(a[0].mean()) < 0.9
    assert torch.equal(a[0], b[0]), 'spikes'
    assert torch.equal(a[3], b[3]) and torch.equal(a[4], b[4]), 'carried states'
    assert_rel(b[1], a[1].cpu(), 'grad z')
    assert_rel(b[2], a[2].cpu(), 'grad weight')


@pytest.mark.parametrize('n,c,t', [(2, 1100, 12), (8, 2048, 24)])
def test_wide_layers_match_the_oracle_and_the_generic_loop(slayer, n, c, t):
    """Layers beyond 1024 neurons take the launch-per-step kernels by themselves."""
    R = slayer.utils.recurrent
    gen = torch.Generator().manual_seed(c + t)
    z = torch.randn(n, c, t, generator=gen)
    neurons = [base._neuron(slayer) for _ in range(2)]
    syns = [base._Dense(c, torch.Generator().manual_seed(5)).to(dev()) for _ in range(2)]
    for s, nrn in zip(syns, neurons):
        with torch.no_grad():
            s.weight.mul_(6.0 / c ** 0.5)
        s.pre_hook_fx = nrn.quantize_8bit
    assert R._fusable(z.to(dev()), neurons[0]) and R._by_steps(c)
    zs = [z.to(dev()).requires_grad_() for _ in range(2)]
    out = R.custom_recurrent(zs[0], neurons[0], syns[0])
    ref = R.CustomRecurrent.apply(zs[1], neurons[1], R._recurrent_matrix(syns[1]))           # generic loop
    assert 0.01 < float(out.detach().mean()) < 0.9
    assert torch.equal(out.detach(), ref.detach()), 'forward differs from the generic loop'
    rec = neurons[0].quantize_8bit(syns[0].weight.detach().reshape(c, c)).cpu()
    d_i, d_v = neurons[0].current_decay.detach().round().cpu(), neurons[0].voltage_decay.detach().round().cpu()
    thr = neurons[0].threshold + neurons[0].threshold_eps
    zero = torch.tensor([0.0])
    r_spk, r_vol, r_cs, r_vs = O.recurrent_cuba_fwd(z, rec, d_i, d_v, zero, zero, 4096, thr)
    assert_exact(out, r_spk, 'recurrent spikes')
    assert_exact(neurons[0].current_state, r_cs, 'carried current')
    assert_exact(neurons[0].voltage_state, r_vs, 'carried voltage')
    g = torch.rand(n, c, t, generator=gen).to(dev())
    out.backward(g)
    ref.backward(g)
    assert_rel(zs[0].grad, zs[1].grad.cpu(), 'grad z vs generic loop')
    assert_rel(syns[0].weight.grad, syns[1].weight.grad.cpu(), 'grad weight vs generic loop')
    r_gz, _ = O.recurrent_cuba_bwd(g.cpu(), r_spk, r_vol, rec, thr, neurons[0].tau_rho * 100, neurons[0].scale_rho * 0.1)
    assert_rel(zs[0].grad, r_gz, 'grad z vs oracle')


def test_sizes_the_step_kernels_refuse(slayer):
    from lava_dl_amd.slayer import _native as N
    lib = N.lib()
    base_floats = 4 * 2 * 2048 + 2048 * 2048 + 2 * 2048 * 16            # states, packed weights, packed spikes twice
    assert lib.slayer_recurrent_steps_workspace(2, 2048, 10, 0) == 3 * 2 * 2048 * 10 + base_floats
    assert lib.slayer_recurrent_steps_workspace(2, 2048, 10, 1) == 4 * 2 * 2048 * 10 + base_floats
    assert lib.slayer_recurrent_steps_workspace(2, 2050, 10, 0) == -3          # not whole quads of neurons
    assert lib.slayer_recurrent_steps_workspace(2, 16388, 10, 0) == -3
    R = slayer.utils.recurrent
    z = torch.zeros(2, 1030, 4, device=dev())
    assert not R._fusable(z, base._neuron(slayer)) and R._fusable(z[:, :1028].contiguous(), base._neuron(slayer))
    assert R._by_steps(256) and R._by_steps(1028) and not R._by_steps(252) and not R._by_steps(258)
    # a workspace that is too small is refused before anything is launched
    ws = torch.empty(16, device=dev())
    t = torch.zeros(2 * 1028 * 4, device=dev())
    one = torch.zeros(1, device=dev())
    code = lib.slayer_cuba_recurrent_steps_fwd(
        N.ptr(t), N.ptr(t), N.ptr(t), N.ptr(t), N.ptr(t), N.ptr(torch.zeros(1028 * 1028, device=dev())),
        N.ptr(one), N.ptr(one), N.ptr(one), N.ptr(one), 1.0, 0, 1.0, 64, 2, 1028, 1, 1, 1, 1, 4,
        N.ptr(ws), ws.numel(), N.stream_handle())
    assert code == -3


@pytest.mark.parametrize('c', [24, 260])
def test_recurrent_layer_with_the_dense_synapse_module(slayer, c):
    """The recurrent synapse as the package's own Dense layer (what the reference's Recurrent blocks hold,
    block/cuba.py:166-176): the kernels (one launch for 24 neurons, a launch per step for 260) and the plain loop
    that calls the synapse module step by step give the same spikes and weight gradients."""
    R = slayer.utils.recurrent
    gen = torch.Generator().manual_seed(c)
    n, t = 3, 40
    z = (torch.randn(n, c, t, generator=gen) * 1.5).to(dev())
    g = torch.rand(n, c, t, generator=gen).to(dev())
    results = []
    for loop in (False, True):
        neuron = base._neuron(slayer)
        syn = slayer.synapse.Dense(c, c, pre_hook_fx=neuron.quantize_8bit).to(dev())
        with torch.no_grad():
            syn.weight.copy_((torch.randn(c, c, generator=torch.Generator().manual_seed(5)) * 3.0 / c ** 0.5)
                             .reshape(syn.weight.shape))
        out = R.custom_recurrent_ground_truth_1(z, neuron, syn) if loop else R.custom_recurrent(z, neuron, syn)
        out.backward(g)
        results.append((out.detach(), syn.weight.grad))
    assert 0.01 < float(results[0][0].mean()) < 0.9
    assert torch.equal(results[0][0], results[1][0]), 'spikes'
    assert results[0][1].shape == results[1][1].shape == (c, c, 1, 1, 1)
