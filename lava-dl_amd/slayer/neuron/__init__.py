from . import dynamics, cuba, alif, rf, rf_iz, adrf, adrf_iz, sigma_delta
from . import norm
from .dropout import Dropout

__all__ = ['dynamics', 'cuba', 'alif', 'rf', 'rf_iz', 'adrf', 'adrf_iz', 'sigma_delta', 'norm', 'Dropout']
