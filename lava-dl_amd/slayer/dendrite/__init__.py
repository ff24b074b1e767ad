from .sigma import Sigma

__all__ = ['Sigma']
