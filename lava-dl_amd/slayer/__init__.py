"""MI355X-native drop-in for the hot path of lava.lib.dl.slayer: neuron
dynamics, spike functions, time shift and temporal filter, all backed by
libslayer_hip.so (hand-written HIP for gfx950)."""
from . import neuron, spike, utils, axon, dendrite, block, synapse
from ._native import range_check, range_flag, range_policy, clear_range_flag

__all__ = ['neuron', 'spike', 'utils', 'axon', 'dendrite', 'block', 'synapse',
           'range_check', 'range_flag', 'range_policy', 'clear_range_flag']
