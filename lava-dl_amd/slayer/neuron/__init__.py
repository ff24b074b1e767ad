from . import dynamics, cuba, alif, rf

__all__ = ['dynamics', 'cuba', 'alif', 'rf']
