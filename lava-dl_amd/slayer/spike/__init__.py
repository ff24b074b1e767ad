from .spike import Spike
from . import complex

__all__ = ['Spike', 'complex']
