from . import time, filter, int_utils
from .int_utils import right_shift_to_zero
from .quantize import quantize, MODE

__all__ = ['time', 'filter', 'int_utils', 'right_shift_to_zero', 'quantize', 'MODE']
