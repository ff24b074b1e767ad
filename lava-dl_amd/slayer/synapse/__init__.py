from .layer import Conv, Dense, Pool, conv_synapse

__all__ = ['Conv', 'Dense', 'Pool', 'conv_synapse']
