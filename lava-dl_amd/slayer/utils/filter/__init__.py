from .conv import conv, corr

__all__ = ['conv', 'corr']
