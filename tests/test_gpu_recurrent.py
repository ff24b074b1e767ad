"""Recurrent CUBA layer: the one-launch time loop against the CPU oracle (bit-exact spikes and
voltages with quantised weights), against the loops of one-step neuron calls (the reference's own
check, tests/lava/lib/dl/slayer/utils/test_recurrent.py:101-190), and the fallback for other neurons."""
import pytest
import torch

from oracle import slayer_oracle as O
from tests.util import dev, assert_exact, assert_rel

pytestmark = pytest.mark.gpu


@pytest.fixture(scope='module')
def slayer():
    import lava_dl_amd.slayer as s
    return s


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
    assert_rel(zg.grad, r_gz, 'recurrent grad z', rel=1e-4)
    assert_rel(syn.weight.grad.reshape(c, c), r_gw, 'recurrent grad weight', rel=1e-4)
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
        assert_rel(syns[0].weight.grad.cpu(), syns[i].weight.grad.cpu(), f'weight gradient vs loop {i}', rel=1e-4)


def test_other_neurons_take_the_generic_loop(slayer):
    gen = torch.Generator().manual_seed(7)
    n, c, t = 2, 12, 40
    z = torch.randn(n, c, t, generator=gen).mul(2).to(dev()).requires_grad_()
    mk = lambda: slayer.neuron.alif.Neuron(1.0, 0.5, 0.25, 0.1, 0.1, 0.2, persistent_state=True).to(dev())
    a, b = mk(), mk()
    syn_a, syn_b = (_Dense(c, torch.Generator().manual_seed(3)).to(dev()) for _ in range(2))
    out = slayer.utils.recurrent.custom_recurrent(z, a, syn_a)
    ref = slayer.utils.recurrent.custom_recurrent_ground_truth_2(z.detach(), b, syn_b)
    assert torch.equal(out, ref.detach()) and float(out.detach().sum()) > 0
    out.sum().backward()
    assert torch.isfinite(z.grad).all() and syn_a.weight.grad is not None
