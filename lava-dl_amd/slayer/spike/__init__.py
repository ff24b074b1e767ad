"""Spike functions with surrogate gradients: ``Spike`` for a real state, ``complex.Spike`` for a resonator's
phase crossing."""
from .spike import Spike
from . import complex

__all__ = ['Spike', 'complex']
