"""Hardware view of the neuron parameters (cx_* integers, device_params, neuron_params): host logic,
runs without a GPU.  Expected values are worked out by hand from the definitions in the reference
(neuron/cuba.py:226-272, alif.py:306-381, rf.py:259-325, adrf.py:343-437, sigma_delta.py:141-154)."""
import numpy as np
import pytest
import torch

import lava_dl_amd.slayer as slayer

N = slayer.neuron


def test_cuba_device_params():
    n = N.cuba.Neuron(threshold=1.25, current_decay=0.25, voltage_decay=0.03, scale=64)
    assert n.device_params == {'type': 'CUBA', 'iDecay': 1024, 'vDecay': 123, 'vThMant': 80, 'refDelay': 1,
                               'gradedSpike': False}
    assert n.scale == 64 and n.weight_exponent == 0 and n.v_th_mant == 80
    assert n.threshold == 1.25 and n.threshold_eps == 0.01 / 4096
    back = N.cuba.neuron_params(n.device_params)
    assert back == {'threshold': 1.25, 'current_decay': 0.25, 'voltage_decay': 123 / 4096}
    assert N.cuba.Neuron(**back).device_params == n.device_params


def test_cuba_threshold_is_truncated_to_the_weight_grid_and_decays_are_clamped():
    n = N.cuba.Neuron(threshold=1.26, current_decay=1.5, voltage_decay=-0.2, scale=64)
    assert n.threshold == 80 / 64 and n.v_th_mant == 80
    assert n.cx_current_decay == 4096 and n.cx_voltage_decay == 0


def test_cuba_per_channel_decays_are_arrays_inside_their_range():
    n = N.cuba.Neuron(threshold=1.0, current_decay=[0.1, 0.3], voltage_decay=0.5, shared_param=False)
    assert n.cx_current_decay == round(0.1 * 4096)              # before the first input: the range minimum
    torch.manual_seed(3)
    n.shape, n.num_neurons = (5,), 5
    n._draw_per_channel(5, n.device)
    cur, vol = n.cx_current_decay, n.cx_voltage_decay
    assert cur.shape == (5,) and cur.dtype.kind == 'i' and len(set(cur.tolist())) > 1
    assert (cur >= round(0.1 * 4096)).all() and (cur <= round(0.3 * 4096)).all()
    assert (vol >= int(0.5 * 0.99 * 4096)).all() and (vol <= round(0.5 * 1.01 * 4096)).all()


def test_alif_device_params():
    n = N.alif.Neuron(threshold=1.0, threshold_step=0.51, current_decay=0.5, voltage_decay=0.125,
                      threshold_decay=0.1, refractory_decay=0.2, graded_spike=True)
    want = {'type': 'ALIF', 'iDecay': 2048, 'vDecay': 512, 'thDecay': 410, 'refDecay': 819, 'vThMant': 64,
            'vThStep': 32, 'refDelay': 1, 'gradedSpike': True}
    assert n.device_params == want
    assert n.threshold_step == 32 / 64
    back = N.alif.neuron_params(want)
    assert back['threshold'] == 1.0 and back['threshold_step'] == 1.0       # the reference reads vThMant for both
    assert back['threshold_decay'] == 410 / 4096 and back['refractory_decay'] == 819 / 4096


@pytest.mark.parametrize('module,kind', [(N.rf, 'RF_PHASE'), (N.rf_iz, 'RF_IZHIKEVICH')])
def test_resonator_device_params(module, kind):
    n = module.Neuron(threshold=1.0, period=16, decay=0.05)
    sin = int(round(4096 * np.sin(2 * np.pi / 16) * 0.95))
    cos = int(round(4096 * np.cos(2 * np.pi / 16) * 0.95))
    assert n.device_params == {'type': kind, 'sinDecay': sin, 'cosDecay': cos, 'vThMant': 64, 'gradedSpike': False}
    assert abs(float(n.period[0]) - 16) < 0.01 and abs(float(n.decay[0]) - 0.05) < 1e-3
    assert abs(float(n.frequency[0]) - 1 / 16) < 1e-4 and abs(float(n.lam[0]) + np.log(0.95)) < 1e-3
    back = module.neuron_params(n.device_params)
    again = module.Neuron(**back)
    assert again.cx_sin_decay == sin and again.cx_cos_decay == cos


def test_resonator_clamp_keeps_the_gain_below_one():
    n = N.rf.Neuron(threshold=1.0, period=4, decay=0.0)          # sin = 4096, cos = 0 before the clamp
    assert n.cx_sin_decay == 4095 and n.cx_cos_decay == 0
    with pytest.raises(AssertionError):
        N.rf.Neuron(threshold=1.0, period=3, decay=0.1)


@pytest.mark.parametrize('module,kind', [(N.adrf, 'ADRF_PHASE'), (N.adrf_iz, 'ADRF_IZHIKEVICH')])
def test_adaptive_resonator_device_params(module, kind):
    n = module.Neuron(threshold=1.0, threshold_step=0.25, period=10, decay=0.1, threshold_decay=0.05,
                      refractory_decay=0.5)
    p = n.device_params
    assert p['type'] == kind and p['vThMant'] == 64 and p['vThStep'] == 16
    assert p['thDecay'] == 205 and p['refDecay'] == 2048
    assert p['sinDecay'] == int(round(4096 * np.sin(2 * np.pi / 10) * 0.9))
    assert set(p) == {'type', 'sinDecay', 'cosDecay', 'thDecay', 'refDecay', 'vThMant', 'vThStep', 'gradedSpike'}
    back = module.neuron_params(p)
    assert set(back) == {'threshold', 'threshold_step', 'period', 'decay', 'threshold_decay', 'refractory_decay'}
    assert module.Neuron(**back).cx_refractory_decay == 2048


def test_sigma_delta_device_params():
    n = N.sigma_delta.Neuron(threshold=0.1, activation=torch.relu)
    assert n.device_params == {'type': 'SDNN', 'activation': 'relu', 'vThMant': 6}
    assert N.sigma_delta.neuron_params(n.device_params) == {'threshold': 6 / 64}
    assert n.scale == 64


def test_small_utilities():
    U = slayer.utils
    w = torch.tensor([-9.0, -4.001, -0.02, 0.017, 0.05, 3.97, 9.0])
    q = U.quantize_hook_fx(w)
    assert torch.equal(q, torch.tensor([-8.0, -4.0, -0.03125, 0.03125, 0.0625, 3.96875, 7.96875]))      # limits -512 / 64 and 510 / 64
    assert torch.equal(U.quantize_hook_fx(w, descale=True), q * 64)
    assert torch.equal(U.quantize_hook_fx(torch.tensor([1.0, -1.0]), scale=4, num_bits=1), torch.tensor([0.5, -1.0]))
    x = torch.tensor([-2.7, -0.3, 0.0, 0.9, 5.5], requires_grad=True)
    y = U.int_utils.Q2Zero.apply(x)
    assert torch.equal(y.detach(), torch.tensor([-2.0, 0.0, 0.0, 0.0, 5.0]))
    y.sum().backward()
    assert torch.equal(x.grad, torch.ones(5))
    r = U.time.replicate(torch.arange(6.0).reshape(2, 3), 4)
    assert r.shape == (2, 3, 4) and all(torch.equal(r[..., t], torch.arange(6.0).reshape(2, 3)) for t in range(4))
    m = U.diagonal_mask(5, 3)
    assert torch.equal(m, (torch.eye(5) + torch.diag(torch.ones(4), 1) + torch.diag(torch.ones(4), -1)))
    assert torch.equal(U.diagonal_mask(4, 1), torch.eye(4)) and torch.equal(U.diagonal_mask(4, 2), U.diagonal_mask(4, 3))
    with pytest.raises(Exception):
        U.diagonal_mask(4, 0)
    e = torch.tensor([[1.0, 0.0, -2.0, 0.0, 0.0], [3.0, 0.0, 0.0, 0.0, 1.0]])
    assert abs(U.event_rate(e) - 2 / 8) < 1e-7 and U.event_rate(e[:, :1]) == 1.0
    d = U.dotdict(a=1)
    d.b = 2
    assert d['b'] == 2 and d.a == 1 and d.missing is None

    class Handle:
        @U.staticproperty
        def value():
            return 42
    assert Handle.value == 42


def test_mean_only_batch_norm():
    """Batch statistics while training, running mean otherwise; hand-computed expectations
    (neuron/norm.py:9-95 in the reference)."""
    norm = N.norm.MeanOnlyBatchNorm(momentum=0.25)
    x = torch.arange(2 * 3 * 4, dtype=torch.float32).reshape(2, 3, 4)
    mean = torch.tensor([7.5, 11.5, 15.5])                     # per feature over batch and time
    norm.train()
    assert torch.allclose(norm(x), x - mean.reshape(1, 3, 1))
    assert norm.num_features == 3 and torch.allclose(norm.running_mean, 0.25 * mean)
    norm.eval()
    assert torch.allclose(norm(x), x - 0.25 * mean.reshape(1, 3, 1))
    assert torch.allclose(norm.running_mean, 0.25 * mean)      # no update outside training
    norm.train()
    norm.update = False
    assert torch.allclose(norm(x), x - 0.25 * mean.reshape(1, 3, 1))
    y5 = N.norm.MeanOnlyBatchNorm()(torch.ones(2, 3, 2, 2, 5))
    assert y5.shape == (2, 3, 2, 2, 5) and float(y5.abs().max()) == 0.0
    with pytest.raises(AssertionError):
        N.norm.MeanOnlyBatchNorm()(torch.ones(1, 2, 1, 1, 1, 3))


def test_weight_scale_batch_norm():
    norm = N.norm.WgtScaleBatchNorm(momentum=0.5, weight_exp_bits=3)
    gen = torch.Generator().manual_seed(5)
    x = 5.0 * torch.randn(4, 6, 50, generator=gen) + 2.0
    norm.train()
    y = norm(x)
    mean = x.transpose(0, 1).reshape(6, -1).mean(dim=1)
    var = x.var(unbiased=False)
    scale = 2.0 ** float(torch.ceil(torch.log2(torch.sqrt(var + 1e-5))).clamp(-3, 3))
    assert scale == 8.0                                         # std ~ 5 rounds up to 2**3
    assert torch.allclose(y, (x - mean.reshape(1, 6, 1)) / scale, atol=1e-6)
    n = x.numel() / 6
    assert torch.allclose(norm.running_var, 0.5 * var * n / (n + 1))
    assert torch.allclose(norm.running_mean, 0.5 * mean)
    assert float(norm.weight_exp) == float(torch.ceil(torch.log2(torch.sqrt(norm.running_var + 1e-5))))
    assert float(norm.std(torch.tensor([1.0e6]))) == 8.0 and float(norm.std(torch.tensor([1.0e-9]))) == 0.125
    norm.eval()
    y = norm(x)
    assert torch.allclose(y, (x - 0.5 * mean.reshape(1, 6, 1)) / float(norm.std(norm.running_var)), atol=1e-6)


def test_neuron_hooks_its_quantiser_into_the_norm():
    n = N.cuba.Neuron(1.0, 0.25, 0.03, norm=N.norm.MeanOnlyBatchNorm)
    assert n.norm.pre_hook_fx == n.quantize_8bit
    n.norm.running_mean = torch.tensor([0.26, -0.51])
    assert torch.equal(n.norm.bias, -torch.tensor([0.25, -0.5]) * 64)      # steps of 2 / 64, descaled
    r = N.rf.Neuron(1.0, 10, 0.1, norm=N.norm.WgtScaleBatchNorm)
    assert r.norm is None and r.real_norm.pre_hook_fx == r.quantize_8bit and r.imag_norm is not r.real_norm

    class Plain(torch.nn.Module):
        def forward(self, x):
            return x
    assert isinstance(N.cuba.Neuron(1.0, 0.25, 0.03, norm=Plain).norm, Plain)


def test_neuron_dropout_drops_whole_neurons():
    drop = N.Dropout(0.5)
    torch.manual_seed(0)
    x = torch.ones(8, 4, 5, 20)
    y = drop(x)
    assert y.shape == x.shape
    per_neuron = y.reshape(8 * 4 * 5, 20)
    assert bool(((per_neuron == 0).all(dim=1) | (per_neuron == 2).all(dim=1)).all())      # constant over time
    assert 0 < float((per_neuron[:, 0] == 0).float().mean()) < 1
    drop.eval()
    assert torch.equal(drop(x), x)
