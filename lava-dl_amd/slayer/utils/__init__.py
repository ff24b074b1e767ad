from . import time, filter, int_utils, recurrent
from .int_utils import right_shift_to_zero
from .quantize import quantize, quantize_hook_fx, MODE
from .quantize import MODE as QUANTIZE_MODE
from .utils import staticproperty, diagonal_mask, event_rate, dotdict

__all__ = ['time', 'filter', 'int_utils', 'recurrent', 'right_shift_to_zero', 'quantize', 'quantize_hook_fx',
           'MODE', 'QUANTIZE_MODE', 'staticproperty', 'diagonal_mask', 'event_rate', 'dotdict']
