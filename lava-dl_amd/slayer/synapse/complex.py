"""Complex synapses (synapse/complex.py in the reference): a real and an imaginary synapse of the same kind
applied to the same spikes, for the neurons with complex dynamics (resonate-and-fire and its adaptive forms)."""
import numpy as np
import torch

from . import layer


class ComplexLayer(torch.nn.Module):
    """A pair of synapses; ``forward`` returns ``(real(input), imag(input))`` (synapse/complex.py:11-61)."""

    def __init__(self):
        super().__init__()
        self.real = lambda x: x
        self.imag = lambda x: x
        self.complex = True

    def forward(self, input):
        return self.real(input), self.imag(input)

    def enable_weight_norm(self):
        self.real.enable_weight_norm()
        self.imag.enable_weight_norm()

    def disable_weight_norm(self):
        self.real.disable_weight_norm()
        self.imag.disable_weight_norm()

    @property
    def grad_norm(self):
        return np.sqrt(self.real.grad_norm ** 2 + self.imag.grad_norm ** 2)

    @property
    def pre_hook_fx(self):
        if self.real.pre_hook_fx is not self.imag.pre_hook_fx:
            raise Exception('Quantization method of real and imaginary weights must be same.')
        return self.real.pre_hook_fx

    @pre_hook_fx.setter
    def pre_hook_fx(self, fx):
        self.real.pre_hook_fx = fx
        self.imag.pre_hook_fx = fx

    @property
    def shape(self):
        return self.real.shape


def _pair_of(kind, doc):
    def __init__(self, *args, **kwargs):
        ComplexLayer.__init__(self)
        self.real = kind(*args, **kwargs)
        self.imag = kind(*args, **kwargs)
        self.in_channels, self.out_channels = self.real.in_channels, self.real.out_channels
        self.weight_norm_enabled = self.real.weight_norm_enabled
    return type(kind.__name__, (ComplexLayer,), {'__init__': __init__, '__doc__': doc, '__module__': __name__})


Dense = _pair_of(layer.Dense, 'Dense complex synapse (synapse/complex.py:64-110): arguments of synapse.Dense.')
Conv = _pair_of(layer.Conv, 'Convolution complex synapse (synapse/complex.py:113-174): arguments of synapse.Conv.')
Pool = _pair_of(layer.Pool, 'Pooling complex synapse (synapse/complex.py:177-230): arguments of synapse.Pool.')
ConvTranspose = _pair_of(layer.ConvTranspose,
                         'Transposed convolution complex synapse (synapse/complex.py:233-296): arguments of '
                         'synapse.ConvTranspose.')
Unpool = _pair_of(layer.Unpool, 'Unpooling complex synapse (synapse/complex.py:299-356): arguments of synapse.Unpool.')
