from .replicate import replicate
from .shift import shift

__all__ = ['replicate', 'shift']
