from .layer import Conv, Dense, conv_synapse

__all__ = ['Conv', 'Dense', 'conv_synapse']
