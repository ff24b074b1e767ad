"""Neuron modules on the GPU dynamics kernels: one module per neuron model (each with a ``Neuron`` class
and ``neuron_params``), the dynamics operators they are built from, and the norm / dropout helpers a neuron
can be given."""
from . import dynamics, cuba, alif, rf, rf_iz, adrf, adrf_iz, sigma_delta
from . import norm
from .dropout import Dropout

__all__ = ['dynamics', 'cuba', 'alif', 'rf', 'rf_iz', 'adrf', 'adrf_iz', 'sigma_delta', 'norm', 'Dropout']
