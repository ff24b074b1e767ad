"""Sigma-delta neuron on the GPU kernels (counterpart of neuron/sigma_delta.py in the reference:
constructor :68-118, forward :179-219): running sum of the incoming events, activation, delta
encoding of the result."""
import torch

from .base import Neuron as _Base
from ..axon.delta import Delta
from ..dendrite.sigma import Sigma


def neuron_params(device_params, scale=1 << 6):
    """Constructor arguments from a hardware parameter dictionary (neuron/sigma_delta.py:15-33)."""
    return {'threshold': device_params['vThMant'] / scale}


class Neuron(_Base):
    """``Neuron(threshold, activation, ...)``: ``delta(activation(sigma(input) [+ bias]))``; the
    output events are graded.  ``set_bias`` adds a per-neuron bias before the activation."""

    def __init__(self, threshold, activation, tau_grad=1, scale_grad=1, scale=1 << 6, cum_error=False,
                 norm=None, dropout=None, shared_param=True, persistent_state=False, requires_grad=False):
        super().__init__(threshold, tau_grad, scale_grad, scale, norm, dropout, shared_param,
                         persistent_state, requires_grad, graded_spike=True)
        self.activation = activation
        self.sigma = Sigma(persistent_state=persistent_state)
        self.delta = Delta(threshold=self._threshold, scale=self.s_scale, tau_grad=tau_grad, scale_grad=scale_grad,
                           cum_error=cum_error, shared_param=shared_param, persistent_state=persistent_state,
                           requires_grad=requires_grad)
        self.bias_is_set = False
        self.register_parameter('bias', torch.nn.Parameter(torch.FloatTensor([0]), requires_grad=requires_grad))

    @property
    def device(self):
        return self.delta.pre_state.device

    @property
    def threshold(self):
        return self.delta.threshold

    @property
    def device_params(self):
        return {
            'type': 'SDNN',
            'activation': self.activation.__name__,
            'vThMant': self.v_th_mant,
        }

    def set_bias(self, bias):
        self.bias.data = (bias if self.shape is None else bias.reshape(self.shape)).to(self.bias.device)
        self.bias_is_set = True

    def forward(self, input):
        dend = self.sigma(input)
        if self.norm is not None:
            dend = self.norm(dend)
        if self.bias_is_set:
            dend = dend + torch.unsqueeze(torch.unsqueeze(self.bias, dim=0), dim=-1)
        axon = self.delta(self.activation(dend))
        if self.drop is not None:
            axon = self.drop(axon)
        if self.shape is None:
            if self.sigma.shape != self.delta.shape:
                raise AssertionError('The shape of sigma and delta do not match. '
                                     f'Found {self.sigma.shape=} and {self.delta.shape=}.')
            self.shape = self.sigma.shape
        return axon
