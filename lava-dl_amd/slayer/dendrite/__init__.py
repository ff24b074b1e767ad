"""What sits on a neuron's input: the running sum that decodes delta events."""
from .sigma import Sigma

__all__ = ['Sigma']
