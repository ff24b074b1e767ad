"""Resonate-and-fire neuron on the GPU dynamics kernels
(counterpart of neuron/rf.py in the reference: parameters :136-257, call order :429-471)."""
import numpy as np
import torch

from .base import Neuron as _Base, hardware_decay
from .dynamics import resonator, rf_fused
from .dynamics import delays as D
from ..spike import complex as complex_spike
from ..utils.quantize import quantize

TAU_RHO_MULT = 0.5      # surrogate-gradient constants of the RF family (neuron/rf.py:19-20)
SCALE_RHO_MULT = 10


def neuron_params(device_params, scale=1 << 6, p_scale=1 << 12):
    """Constructor arguments from a hardware parameter dictionary (neuron/rf.py:23-50)."""
    sin_decay = device_params['sinDecay'] / p_scale
    cos_decay = device_params['cosDecay'] / p_scale
    return {
        'threshold': device_params['vThMant'] / scale,
        'period': 1 / (np.arctan2(sin_decay, cos_decay) / 2 / np.pi),
        'decay': 1 - np.sqrt(sin_decay ** 2 + cos_decay ** 2),
    }


class ResonatorNeuron(_Base):
    """What the resonator family shares (rf, rf_iz, adrf, adrf_iz in the reference): the rotation
    parameters sin_decay / cos_decay from (period, decay), their clamp to the first quadrant of the
    unit circle, per-channel initialisation, one norm per input component, and the complex state."""

    def __init__(self, threshold, period, decay, tau_grad=1, scale_grad=1, scale=1 << 6, norm=None,
                 dropout=None, shared_param=True, persistent_state=False, requires_grad=False,
                 graded_spike=False, log_init=True, extra_decays=None, extra_states=None):
        super().__init__(threshold, tau_grad, scale_grad, scale, None, dropout, shared_param,
                         persistent_state, requires_grad, graded_spike)
        self.real_norm = self._make_norm(norm)
        self.imag_norm = self._make_norm(norm)
        self.log_init = log_init

        def check(p):
            if p < 4:
                raise AssertionError(f'Neuron period less than 4 does not make sense. Found period={p}.')

        if shared_param:
            if not np.isscalar(decay) or not np.isscalar(period):
                raise AssertionError('Expected period and decay to be scalars when shared_param is True. '
                                     f'Found {period=}, {decay=}.')
            check(period)
            start_p, start_d = period, decay
        else:
            pr = (period * 0.99, period * 1.01) if np.isscalar(period) else tuple(period)
            dr = (decay * 0.99, decay * 1.01) if np.isscalar(decay) else tuple(decay)
            if len(pr) != 2 or len(dr) != 2:
                raise AssertionError(f'Expected [min, max] ranges. Found {period=}, {decay=}.')
            check(period if np.isscalar(period) else min(period))
            self._period_range, self._decay_range = pr, dr
            start_p, start_d = pr[0], dr[0]
        for name, fn in (('sin_decay', np.sin), ('cos_decay', np.cos)):
            value = self.p_scale * fn(2 * np.pi / start_p) * (1 - start_d)
            self.register_parameter(name, torch.nn.Parameter(torch.FloatTensor([value]),
                                                             requires_grad=self.requires_grad))
        if extra_decays:
            self._register_decays(**extra_decays)
        self._register_states(real_state=0.0, imag_state=0.0, **(extra_states or {}))
        self.clamp()

    def clamp(self):
        """Keep the gain below 1 (4095/4096), sin_decay >= 1 and cos_decay >= 0 (and the other
        decays inside [0, 1])."""
        with torch.no_grad():
            for name, prm in self.named_parameters(recurse=False):
                if name not in ('sin_decay', 'cos_decay'):
                    prm.data.clamp_(0, self.p_scale)
            gain = torch.sqrt(self.sin_decay ** 2 + self.cos_decay ** 2)
            ratio = gain.clamp(0, self.p_scale - 1) / gain
            self.sin_decay.data *= ratio
            self.cos_decay.data *= ratio
            self.sin_decay.data.clamp_(1)
            self.cos_decay.data.clamp_(0)

    DEVICE_TYPE = None
    cx_sin_decay = hardware_decay('sin_decay')
    cx_cos_decay = hardware_decay('cos_decay')

    @property
    def decay(self):
        """1 - gain per step, from the rounded rotation parameters."""
        self.clamp()
        s = quantize(self.sin_decay).cpu().data.numpy() / self.p_scale
        c = quantize(self.cos_decay).cpu().data.numpy() / self.p_scale
        return 1 - np.sqrt(s ** 2 + c ** 2)

    @property
    def lam(self):
        return -np.log(1 - self.decay)

    @property
    def frequency(self):
        """Rotations per step."""
        self.clamp()
        return np.arctan2(quantize(self.sin_decay).cpu().data.numpy(),
                          quantize(self.cos_decay).cpu().data.numpy()) / 2 / np.pi

    @property
    def period(self):
        return 1 / self.frequency

    @property
    def device_params(self):
        return {
            'type': self.DEVICE_TYPE,
            'sinDecay': self.cx_sin_decay,
            'cosDecay': self.cx_cos_decay,
            'vThMant': self.v_th_mant,
            'gradedSpike': self.graded_spike,
        }

    def _draw_per_channel(self, channels, device):
        (p_lo, p_hi), (d_lo, d_hi) = self._period_range, self._decay_range
        if self.log_init:
            frequency = torch.logspace(-np.log10(p_hi), -np.log10(p_lo), steps=channels).to(device)
        else:
            frequency = (1 / p_hi + (1 / p_lo - 1 / p_hi) * torch.rand(channels, dtype=torch.float)).to(device)
        decay = d_lo + (d_hi - d_lo) * torch.rand(channels, dtype=torch.float).to(device)
        self.sin_decay.data = self.p_scale * torch.sin(2 * np.pi * frequency) * (1 - decay)
        self.cos_decay.data = self.p_scale * torch.cos(2 * np.pi * frequency) * (1 - decay)
        super()._draw_per_channel(channels, device)          # the other decays, if any

    def _inputs(self, input):
        """Shape checks, state preparation and input norms; returns (real_input, imag_input)."""
        real_input, imag_input = input
        if real_input.shape != imag_input.shape:
            raise AssertionError(f'Real input tensor shape ({real_input.shape}) does not match '
                                 f'with imaginary input shape ({imag_input.shape}).')
        self._prepare(real_input)
        if self.real_norm is not None:
            real_input = self.real_norm(real_input)
        if self.imag_norm is not None:
            imag_input = self.imag_norm(imag_input)
        return real_input, imag_input

    def forward(self, input):
        return self.spike(*self.dynamics(input))


class Neuron(ResonatorNeuron):
    """``Neuron(threshold, period, decay, ...)``: the state rotates by 2 pi / period per step and
    shrinks by (1 - decay); it spikes when the real part is above threshold while the imaginary
    part crosses zero upwards.  ``forward((real_input, imag_input))`` returns the spikes."""
    DEVICE_TYPE = 'RF_PHASE'

    def dynamics(self, input):
        """(real, imag) traces for ``input = (real_input, imag_input)``."""
        real_input, imag_input = self._inputs(input)
        real, imag = resonator.dynamics(real_input, imag_input, quantize(self.sin_decay), quantize(self.cos_decay),
                                        self.real_state, self.imag_state, self.s_scale, debug=self.debug)
        if self.persistent_state:
            with torch.no_grad():
                self.real_state = real[..., -1].clone()
        return real, imag

    def spike(self, real, imag):
        spike = complex_spike.Spike.apply(real, imag, self.threshold, self.tau_rho * TAU_RHO_MULT,
                                          self.scale_rho * SCALE_RHO_MULT, self.graded_spike, self.imag_state, 1)
        if self.persistent_state:
            with torch.no_grad():
                self.imag_state = imag[..., -1].clone()
        if self.drop is not None:
            spike = self.drop(spike)
        return spike

    def forward(self, input, delays=None):
        """Spike response to ``(real_input, imag_input)``.  Without input normalisation the dynamics
        and the spike run as one fused kernel per direction (same bits as ``spike(*dynamics(input))``).
        ``delays`` (its input shift applies to both inputs) and ``debug``: as in ``cuba.Neuron.forward``."""
        if self.real_norm is not None or self.imag_norm is not None or self.debug or (delays and self.drop is not None):
            real, imag = self.dynamics((D.chain_input(delays, input[0]), D.chain_input(delays, input[1])))
            spike = self.spike(real, imag)
            if delays:
                self.spike_last = spike[..., -1].detach().clone()
            return D.chain_output(delays, spike)
        real_input, imag_input = input
        if real_input.shape != imag_input.shape:
            raise AssertionError(f'Real input tensor shape ({real_input.shape}) does not match '
                                 f'with imaginary input shape ({imag_input.shape}).')
        self._prepare(real_input)
        args = (real_input, imag_input, quantize(self.sin_decay), quantize(self.cos_decay),
                self.real_state, self.imag_state, self.imag_state, self.s_scale, self.threshold)
        needs_grad = (real_input.requires_grad or imag_input.requires_grad or self.requires_grad
                      or D.needs_grad(delays))
        if not (torch.is_grad_enabled() and needs_grad):
            # nothing to differentiate: only the spikes are written, the last state comes per neuron
            real_last, imag_last, spike, *rest = rf_fused.spikes(*args, self.graded_spike, 1, delays=delays)
        else:
            real, imag, spike, *rest = rf_fused.dynamics(*args, self.tau_rho * TAU_RHO_MULT,
                                                         self.scale_rho * SCALE_RHO_MULT, self.graded_spike, 1,
                                                         delays=delays)
            real_last, imag_last = real[..., -1], imag[..., -1]
        if delays:
            self.spike_last = rest[0]
        if self.persistent_state:
            with torch.no_grad():
                self._carry(real_state=real_last, imag_state=imag_last)
        if self.drop is not None:
            spike = self.drop(spike)
        return spike
