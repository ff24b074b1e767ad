from . import time, filter, int_utils, recurrent
from .int_utils import right_shift_to_zero
from .quantize import quantize, MODE

__all__ = ['time', 'filter', 'int_utils', 'recurrent', 'right_shift_to_zero', 'quantize', 'MODE']
