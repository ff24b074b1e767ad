from .layer import Conv, conv_synapse

__all__ = ['Conv', 'conv_synapse']
