"""Adaptive leaky integrate-and-fire neuron on the GPU dynamics kernels
(counterpart of neuron/alif.py in the reference: call order :499-525, spike :557-591)."""
import torch

from .base import Neuron as _Base, hardware_decay
from .dynamics import leaky_integrator, adaptive_threshold, alif_fused
from .dynamics import delays as D
from ..spike import Spike

TAU_RHO_MULT = 100
SCALE_RHO_MULT = 0.1


def neuron_params(device_params, scale=1 << 6, p_scale=1 << 12):
    """Constructor arguments from a hardware parameter dictionary (neuron/alif.py:26-52; the step
    is read from the threshold mantissa there as well)."""
    return {
        'threshold': device_params['vThMant'] / scale,
        'threshold_step': device_params['vThMant'] / scale,
        'current_decay': device_params['iDecay'] / p_scale,
        'voltage_decay': device_params['vDecay'] / p_scale,
        'threshold_decay': device_params['thDecay'] / p_scale,
        'refractory_decay': device_params['refDecay'] / p_scale,
    }


class Neuron(_Base):
    """``Neuron(threshold, threshold_step, current_decay, voltage_decay, threshold_decay,
    refractory_decay, ...)``.  The voltage is not reset; a spike raises the threshold by
    ``threshold_step`` and the refractory state by twice the threshold."""

    def __init__(self, threshold, threshold_step, current_decay, voltage_decay, threshold_decay,
                 refractory_decay, tau_grad=1, scale_grad=1, scale=1 << 6, norm=None, dropout=None,
                 shared_param=True, persistent_state=False, requires_grad=False, graded_spike=False):
        super().__init__(threshold, tau_grad, scale_grad, scale, norm, dropout, shared_param,
                         persistent_state, requires_grad, graded_spike)
        self.threshold_step = int(threshold_step * self.w_scale) / self.w_scale
        self._register_decays(current_decay=current_decay, voltage_decay=voltage_decay,
                              threshold_decay=threshold_decay, refractory_decay=refractory_decay)
        self._register_states(current_state=0.0, voltage_state=0.0,
                              threshold_state=lambda: self.threshold, refractory_state=0.0)
        self.threshold_state.fill_(self.threshold)
        self.clamp()

    cx_current_decay = hardware_decay('current_decay')
    cx_voltage_decay = hardware_decay('voltage_decay')
    cx_threshold_decay = hardware_decay('threshold_decay')
    cx_refractory_decay = hardware_decay('refractory_decay')

    @property
    def v_th_step(self):
        return int(self.threshold_step * self.w_scale)

    @property
    def ref_delay(self):
        return 1

    @property
    def device_params(self):
        return {
            'type': 'ALIF',
            'iDecay': self.cx_current_decay,
            'vDecay': self.cx_voltage_decay,
            'thDecay': self.cx_threshold_decay,
            'refDecay': self.cx_refractory_decay,
            'vThMant': self.v_th_mant,
            'vThStep': self.v_th_step,
            'refDelay': self.ref_delay,
            'gradedSpike': self.graded_spike,
        }

    def dynamics(self, input):
        """(current, voltage, threshold, refractory) traces."""
        self._prepare(input)
        if self.norm is not None:
            input = self.norm(input)
        current = leaky_integrator.dynamics(input, self._q('current_decay'), self.current_state.contiguous(),
                                            self.s_scale, debug=self.debug)
        voltage = leaky_integrator.dynamics(current, self._q('voltage_decay'), self.voltage_state.contiguous(),
                                            self.s_scale, debug=self.debug)
        threshold, refractory = adaptive_threshold.dynamics(
            voltage, self.refractory_state.contiguous(), self._q('refractory_decay'),
            self.threshold_state.contiguous(), self._q('threshold_decay'),
            self.threshold_step, self.threshold, self.s_scale, debug=self.debug)
        if self.persistent_state:
            with torch.no_grad():
                self.current_state = current[..., -1].clone()
                self.voltage_state = voltage[..., -1].clone()
                self.threshold_state = threshold[..., -1].clone()
                self.refractory_state = refractory[..., -1].clone()
        return current, voltage, threshold, refractory

    def spike(self, voltage, threshold, refractory):
        spike = Spike.apply(voltage, threshold + refractory, self.tau_rho * TAU_RHO_MULT,
                            self.scale_rho * SCALE_RHO_MULT, self.graded_spike, self.voltage_state, 1)
        if self.persistent_state:
            with torch.no_grad():
                last = spike[..., -1]
                self.refractory_state = adaptive_threshold.persistent_ref_state(
                    self.refractory_state, last, self.threshold_state).detach().clone()
                self.threshold_state = adaptive_threshold.persistent_th_state(
                    self.threshold_state, last, self.threshold_step).detach().clone()
        if self.drop is not None:
            spike = self.drop(spike)
        return spike

    def forward(self, input, delays=None):
        """Spike response.  Without a norm the whole neuron runs as one fused kernel per direction
        (same bits as ``spike(*dynamics(input)[1:])``).  ``delays`` and ``debug``: as in ``cuba.Neuron.forward``."""
        if self.norm is not None or self.debug or (delays and self.drop is not None):
            _, voltage, threshold, refractory = self.dynamics(D.chain_input(delays, input))
            spike = self.spike(voltage, threshold, refractory)
            if delays:
                self.spike_last = spike[..., -1].detach().clone()
            return D.chain_output(delays, spike)
        self._prepare(input)
        args = (input, self._q('current_decay', True), self._q('voltage_decay', True), self._q('threshold_decay', True),
                self._q('refractory_decay', True), self.current_state, self.voltage_state, self.threshold_state,
                self.refractory_state, self.threshold_step, self.threshold, self.s_scale)
        if not (torch.is_grad_enabled() and (input.requires_grad or self.requires_grad or D.needs_grad(delays))):
            # nothing to differentiate: only the spikes are written, the last states come per neuron
            current_last, voltage_last, _, spike, th_last, ref_last, *rest = alif_fused.spikes(
                *args, self.graded_spike, 1, delays=delays)
        else:
            # without trainable decays the kernel skips the current trace and returns its last step
            current, voltage, _, spike, th_last, ref_last, *rest = alif_fused.dynamics(
                *args, self.tau_rho * TAU_RHO_MULT, self.scale_rho * SCALE_RHO_MULT, self.graded_spike, 1,
                keep_current=self.requires_grad, delays=delays)
            current_last = current[..., -1] if self.requires_grad else current
            voltage_last = voltage[..., -1]
        if delays:
            self.spike_last = rest[0]
        if self.persistent_state:
            with torch.no_grad():
                last = rest[0] if delays else spike[..., -1]
                self._carry(current_state=current_last, voltage_state=voltage_last,
                            refractory_state=adaptive_threshold.persistent_ref_state(ref_last, last, th_last).detach(),
                            threshold_state=adaptive_threshold.persistent_th_state(
                                th_last, last, self.threshold_step).detach())
        if self.drop is not None:
            spike = self.drop(spike)
        return spike
