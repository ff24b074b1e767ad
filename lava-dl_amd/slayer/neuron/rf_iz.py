"""Resonate-and-fire Izhikevich neuron on the GPU dynamics kernels
(counterpart of neuron/rf_iz.py in the reference: call order :433-441, spike :463-489)."""
import torch

from .rf import ResonatorNeuron, neuron_params     # noqa: F401  (same translation as rf)
from .dynamics import resonator
from ..spike import Spike
from ..utils.quantize import quantize

TAU_RHO_MULT = 100      # surrogate-gradient constants (neuron/rf_iz.py:21-22)
SCALE_RHO_MULT = 0.1


class Neuron(ResonatorNeuron):
    """``Neuron(threshold, period, decay, ...)``: a resonator that spikes when its imaginary part
    reaches the threshold; the spike resets the real part to zero and the imaginary part to just
    below the threshold."""
    DEVICE_TYPE = 'RF_IZHIKEVICH'

    def dynamics(self, input):
        """(real, imag) traces for ``input = (real_input, imag_input)``."""
        real_input, imag_input = self._inputs(input)
        real, imag = resonator.dynamics(real_input, imag_input, quantize(self.sin_decay), quantize(self.cos_decay),
                                        self.real_state, self.imag_state, self.s_scale, self.threshold,
                                        debug=self.debug)
        if self.persistent_state:
            with torch.no_grad():
                self.real_state = real[..., -1].clone()
                self.imag_state = imag[..., -1].clone()
        return real, imag

    def spike(self, real, imag):
        spike = Spike.apply(imag, self.threshold, self.tau_rho * TAU_RHO_MULT, self.scale_rho * SCALE_RHO_MULT,
                            self.graded_spike, self.imag_state, 1)
        if self.persistent_state:
            with torch.no_grad():
                last = spike[..., -1]
                self.real_state = resonator.persistent_real_state(self.real_state, last).detach().clone()
                self.imag_state = resonator.persistent_imag_state(
                    self.imag_state, last, self.threshold, self.s_scale).detach().clone()
        if self.drop is not None:
            spike = self.drop(spike)
        return spike
