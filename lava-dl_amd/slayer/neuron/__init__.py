from . import dynamics

__all__ = ['dynamics']
