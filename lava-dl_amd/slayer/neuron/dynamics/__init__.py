from . import leaky_integrator, adaptive_threshold, resonator

__all__ = ['leaky_integrator', 'adaptive_threshold', 'resonator']
