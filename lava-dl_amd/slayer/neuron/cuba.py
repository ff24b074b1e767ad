"""Current-based leaky integrate-and-fire neuron on the GPU dynamics kernels
(counterpart of neuron/cuba.py in the reference: call order :356-374, spike :401-421)."""
import torch

from .base import Neuron as _Base, hardware_decay
from .dynamics import leaky_integrator, cuba_fused
from .dynamics import delays as D
from ..spike import Spike

TAU_RHO_MULT = 100      # surrogate-gradient constants of the CUBA family (neuron/cuba.py:20-21)
SCALE_RHO_MULT = 0.1


def neuron_params(device_params, scale=1 << 6, p_scale=1 << 12):
    """Constructor arguments from a hardware parameter dictionary (neuron/cuba.py:26-49)."""
    return {
        'threshold': device_params['vThMant'] / scale,
        'current_decay': device_params['iDecay'] / p_scale,
        'voltage_decay': device_params['vDecay'] / p_scale,
    }


class Neuron(_Base):
    """``Neuron(threshold, current_decay, voltage_decay, ...)``; decays are fractions of 1
    (stored times 4096), a [min, max] pair draws one value per channel when
    ``shared_param=False``.  ``forward(x)`` returns the spike tensor."""

    def __init__(self, threshold, current_decay, voltage_decay, tau_grad=1, scale_grad=1, scale=1 << 6,
                 norm=None, dropout=None, shared_param=True, persistent_state=False, requires_grad=False,
                 graded_spike=False):
        super().__init__(threshold, tau_grad, scale_grad, scale, norm, dropout, shared_param,
                         persistent_state, requires_grad, graded_spike)
        # the dynamics spike at v >= threshold; hardware spikes at v > threshold
        self.threshold_eps = 0.01 / self.s_scale
        self._register_decays(current_decay=current_decay, voltage_decay=voltage_decay)
        self._register_states(current_state=0.0, voltage_state=0.0)
        self.clamp()

    cx_current_decay = hardware_decay('current_decay')
    cx_voltage_decay = hardware_decay('voltage_decay')

    @property
    def ref_delay(self):
        return 1

    @property
    def device_params(self):
        return {
            'type': 'CUBA',
            'iDecay': self.cx_current_decay,
            'vDecay': self.cx_voltage_decay,
            'vThMant': self.v_th_mant,
            'refDelay': self.ref_delay,
            'gradedSpike': self.graded_spike,
        }

    def dynamics(self, input):
        """(current, voltage) traces; the voltage already carries the reset."""
        self._prepare(input)
        current = leaky_integrator.dynamics(input, self._q('current_decay'), self.current_state.contiguous(),
                                            self.s_scale, debug=self.debug)
        if self.norm is not None:
            current = self.norm(current)
        voltage = leaky_integrator.dynamics(current, self._q('voltage_decay'), self.voltage_state.contiguous(),
                                            self.s_scale, self.threshold + self.threshold_eps, debug=self.debug)
        if self.persistent_state:
            with torch.no_grad():
                self.current_state = current[..., -1].clone()
                self.voltage_state = voltage[..., -1].clone()
        return current, voltage

    def spike(self, voltage):
        spike = Spike.apply(voltage, self.threshold + self.threshold_eps, self.tau_rho * TAU_RHO_MULT,
                            self.scale_rho * SCALE_RHO_MULT, self.graded_spike, self.voltage_state, 1)
        if self.persistent_state:
            with torch.no_grad():
                self.voltage_state = leaky_integrator.persistent_state(
                    self.voltage_state, spike[..., -1]).detach().clone()
        if self.drop is not None:
            spike = self.drop(spike)
        return spike

    def forward(self, input, delays=None):
        """Spike response.  Without a normalisation between current and voltage the three steps run
        as one fused kernel per direction (same bits as ``spike(dynamics(input)[1])``).

        ``delays`` (``dynamics.delays.Delays``) folds a shift of the input and the delays that follow the
        neuron in a block into the same kernels; the result is then the delayed spike tensor and
        ``self.spike_last`` holds the undelayed spike of the last step.  ``debug=True`` takes the separate
        operators (whose ``debug`` cross-checks then run) and so does a neuron with dropout and delays."""
        if self.norm is not None or self.debug or (delays and self.drop is not None):
            _, voltage = self.dynamics(D.chain_input(delays, input))
            spike = self.spike(voltage)
            if delays:
                self.spike_last = spike[..., -1].detach().clone()
            return D.chain_output(delays, spike)
        self._prepare(input)
        args = (input, self._q('current_decay', True), self._q('voltage_decay', True),
                self.current_state.contiguous(), self.voltage_state.contiguous(), self.s_scale,
                self.threshold + self.threshold_eps)
        spike_last = None
        if not (torch.is_grad_enabled() and (input.requires_grad or self.requires_grad
                                             or D.needs_grad(delays))):
            # nothing to differentiate: only the spikes are written, the last current / voltage come per neuron
            current_last, voltage_last, spike, *rest = cuba_fused.spikes(*args, self.graded_spike, 1, delays=delays)
        else:
            # without trainable decays the kernel skips the current trace and returns its last step
            current, voltage, spike, *rest = cuba_fused.dynamics(
                *args, self.tau_rho * TAU_RHO_MULT, self.scale_rho * SCALE_RHO_MULT, self.graded_spike, 1,
                keep_current=self.requires_grad, delays=delays)
            current_last = current[..., -1] if self.requires_grad else current
            voltage_last = voltage[..., -1]
        if delays:
            self.spike_last = spike_last = rest[0]
        if self.persistent_state:
            with torch.no_grad():               # the product below is a new tensor; slices of a trace are copied
                last = spike_last if delays else spike[..., -1]
                self._carry(current_state=current_last,
                            voltage_state=leaky_integrator.persistent_state(voltage_last, last).detach())
        if self.drop is not None:
            spike = self.drop(spike)
        return spike
