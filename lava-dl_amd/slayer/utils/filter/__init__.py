"""Temporal filters: causal convolution and its adjoint."""
from .conv import conv, corr

__all__ = ['conv', 'corr']
