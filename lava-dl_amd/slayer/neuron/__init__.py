from . import dynamics, cuba, alif, rf, rf_iz, adrf, adrf_iz, sigma_delta

__all__ = ['dynamics', 'cuba', 'alif', 'rf', 'rf_iz', 'adrf', 'adrf_iz', 'sigma_delta']
