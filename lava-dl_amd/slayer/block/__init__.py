"""The part of a block's forward pass that follows the synapse: neuron, one-step delay, axonal delay."""
from .base import step_delay, neuron_delay

__all__ = ['step_delay', 'neuron_delay']
