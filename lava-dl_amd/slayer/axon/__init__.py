"""What sits on a neuron's output: the axonal delay (function and learnable module) and the delta encoder."""
from .delay import delay, Delay
from .delta import Delta

__all__ = ['delay', 'Delay', 'Delta']
