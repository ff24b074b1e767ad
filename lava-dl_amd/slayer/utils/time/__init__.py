"""Operations along the time axis (the last one) of ``[N, C, ..., T]`` tensors."""
from .replicate import replicate
from .shift import shift

__all__ = ['replicate', 'shift']
