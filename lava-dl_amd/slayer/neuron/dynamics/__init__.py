"""The fixed-point state recurrences (one module per operator of the reference) and the fused blocks that run
several of them plus the spike function in one kernel."""
from . import (leaky_integrator, adaptive_threshold, resonator, adaptive_phase_th, adaptive_resonator,
               cuba_fused, rf_fused, alif_fused, delays)

__all__ = ['leaky_integrator', 'adaptive_threshold', 'resonator', 'adaptive_phase_th', 'adaptive_resonator',
           'cuba_fused', 'rf_fused', 'alif_fused', 'delays']
