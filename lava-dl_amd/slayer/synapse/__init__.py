from .layer import Conv, ConvTranspose, Dense, Pool, Unpool, conv_synapse, conv_transpose_synapse
from . import complex

__all__ = ['Conv', 'ConvTranspose', 'Dense', 'Pool', 'Unpool', 'complex', 'conv_synapse', 'conv_transpose_synapse']
