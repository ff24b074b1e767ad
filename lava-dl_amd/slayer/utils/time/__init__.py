from .shift import shift

__all__ = ['shift']
