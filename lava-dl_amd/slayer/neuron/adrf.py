"""Adaptive resonate-and-fire neuron (phase threshold) on the GPU dynamics kernels
(counterpart of neuron/adrf.py in the reference: call order :583-611, spike :636-660)."""
import numpy as np
import torch

from .base import hardware_decay
from .rf import ResonatorNeuron
from . import rf as _rf
from .dynamics import resonator, adaptive_phase_th
from ..spike import complex as complex_spike
from ..utils.quantize import quantize

TAU_RHO_MULT = 100      # surrogate-gradient constants (neuron/adrf.py:21-22)
SCALE_RHO_MULT = 0.1


def _exact_range(value):
    """Per-channel ranges of the threshold / refractory decays: a scalar means exactly that value."""
    return [value, value] if np.isscalar(value) else value


def neuron_params(device_params, scale=1 << 6, p_scale=1 << 12):
    """Constructor arguments from a hardware parameter dictionary (neuron/adrf.py:25-55; the step
    is read from the threshold mantissa there as well)."""
    params = _rf.neuron_params(device_params, scale, p_scale)
    return {
        'threshold': params['threshold'],
        'threshold_step': device_params['vThMant'] / scale,
        'period': params['period'],
        'decay': params['decay'],
        'threshold_decay': device_params['thDecay'] / p_scale,
        'refractory_decay': device_params['refDecay'] / p_scale,
    }


class AdaptiveResonatorNeuron(ResonatorNeuron):
    """Parameters and states shared by adrf and adrf_iz: the resonator's, an adaptive threshold
    (rest value ``threshold``, raised by ``threshold_step`` per spike) and a refractory state."""

    def __init__(self, threshold, threshold_step, period, decay, threshold_decay, refractory_decay,
                 tau_grad=1, scale_grad=1, scale=1 << 6, norm=None, dropout=None, shared_param=True,
                 persistent_state=False, requires_grad=False, graded_spike=False, log_init=True):
        if not shared_param:
            threshold_decay, refractory_decay = _exact_range(threshold_decay), _exact_range(refractory_decay)
        super().__init__(threshold, period, decay, tau_grad, scale_grad, scale, norm, dropout, shared_param,
                         persistent_state, requires_grad, graded_spike, log_init,
                         extra_decays=dict(threshold_decay=threshold_decay, refractory_decay=refractory_decay),
                         extra_states=dict(threshold_state=lambda: self.threshold, refractory_state=0.0))
        self.threshold_step = int(threshold_step * self.w_scale) / self.w_scale
        self.threshold_state.fill_(self.threshold)

    cx_threshold_decay = hardware_decay('threshold_decay')
    cx_refractory_decay = hardware_decay('refractory_decay')

    @property
    def v_th_step(self):
        return int(self.threshold_step * self.w_scale)

    @property
    def device_params(self):
        return {
            'type': self.DEVICE_TYPE,
            'sinDecay': self.cx_sin_decay,
            'cosDecay': self.cx_cos_decay,
            'thDecay': self.cx_threshold_decay,
            'refDecay': self.cx_refractory_decay,
            'vThMant': self.v_th_mant,
            'vThStep': self.v_th_step,
            'gradedSpike': self.graded_spike,
        }

    def _spike_updates_adaptation(self, spike):
        last = spike[..., -1]
        self.refractory_state = adaptive_phase_th.persistent_ref_state(
            self.refractory_state, last, self.threshold_state).detach().clone()
        self.threshold_state = adaptive_phase_th.persistent_th_state(
            self.threshold_state, last, self.threshold_step).detach().clone()

    def forward(self, input):
        return self.spike(*self.dynamics(input))


class Neuron(AdaptiveResonatorNeuron):
    """Spikes when the real part reaches threshold + refractory while the imaginary part crosses
    zero upwards; no reset of the resonator state."""
    DEVICE_TYPE = 'ADRF_PHASE'

    def dynamics(self, input):
        """(real, imag, threshold, refractory) traces for ``input = (real_input, imag_input)``."""
        real_input, imag_input = self._inputs(input)
        real, imag = resonator.dynamics(real_input, imag_input, quantize(self.sin_decay), quantize(self.cos_decay),
                                        self.real_state, self.imag_state, self.s_scale, debug=self.debug)
        threshold, refractory = adaptive_phase_th.dynamics(
            real, imag, self.imag_state, self.refractory_state, quantize(self.refractory_decay),
            self.threshold_state, quantize(self.threshold_decay), self.threshold_step, self.threshold,
            self.s_scale, debug=self.debug)
        if self.persistent_state:
            with torch.no_grad():
                self.real_state = real[..., -1].clone()           # the imaginary state is kept until after the spike
                self.threshold_state = threshold[..., -1].clone()
                self.refractory_state = refractory[..., -1].clone()
        return real, imag, threshold, refractory

    def spike(self, real, imag, threshold, refractory):
        spike = complex_spike.Spike.apply(real, imag, threshold + refractory, self.tau_rho * TAU_RHO_MULT,
                                          self.scale_rho * SCALE_RHO_MULT, self.graded_spike, self.imag_state, 1)
        if self.persistent_state:
            with torch.no_grad():
                self.imag_state = imag[..., -1].clone()
                self._spike_updates_adaptation(spike)
        if self.drop is not None:
            spike = self.drop(spike)
        return spike
