"""Adaptive resonate-and-fire Izhikevich neuron on the GPU dynamics kernels
(counterpart of neuron/adrf_iz.py in the reference: call order :574-594, spike :616-645)."""
import torch

from .adrf import AdaptiveResonatorNeuron, neuron_params     # noqa: F401  (same translation as adrf)
from .dynamics import adaptive_resonator
from ..spike import Spike
from ..utils.quantize import quantize

TAU_RHO_MULT = 100      # surrogate-gradient constants (neuron/adrf_iz.py:21-22)
SCALE_RHO_MULT = 0.1


class Neuron(AdaptiveResonatorNeuron):
    """Spikes when the imaginary part reaches threshold + refractory; threshold and refractory adapt
    inside the same recurrence as the resonator (no reset of the resonator state).

    The reference's ``forward`` hands ``spike`` three arguments where it takes four
    (neuron/adrf_iz.py:669-670) and cannot run; here ``forward`` is ``spike(*dynamics(input))``."""
    DEVICE_TYPE = 'ADRF_IZHIKEVICH'

    def dynamics(self, input):
        """(real, imag, threshold, refractory) traces for ``input = (real_input, imag_input)``."""
        real_input, imag_input = self._inputs(input)
        real, imag, threshold, refractory = adaptive_resonator.dynamics(
            real_input, imag_input, quantize(self.sin_decay), quantize(self.cos_decay),
            quantize(self.refractory_decay), quantize(self.threshold_decay),
            self.real_state, self.imag_state, self.refractory_state, self.threshold_state,
            self.threshold_step, self.threshold, self.s_scale, debug=self.debug)
        if self.persistent_state:
            with torch.no_grad():
                self.real_state = real[..., -1].clone()
                self.imag_state = imag[..., -1].clone()
                self.threshold_state = threshold[..., -1].clone()
                self.refractory_state = refractory[..., -1].clone()
        return real, imag, threshold, refractory

    def spike(self, real, imag, threshold, refractory):
        spike = Spike.apply(imag, threshold + refractory, self.tau_rho * TAU_RHO_MULT,
                            self.scale_rho * SCALE_RHO_MULT, self.graded_spike, self.imag_state, 1)
        if self.persistent_state:
            with torch.no_grad():
                self._spike_updates_adaptation(spike)
        if self.drop is not None:
            spike = self.drop(spike)
        return spike
