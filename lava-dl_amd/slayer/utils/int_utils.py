"""Integer helpers that define the rounding rule of the fixed-point dynamics
(utils/int_utils.py:9-31 in the reference)."""
import torch


def right_shift_to_zero(x, bits):
    """``x >> bits`` rounded toward zero for int32/int64 tensors (an arithmetic
    shift alone rounds toward minus infinity)."""
    if x.dtype not in (torch.int32, torch.int64):
        raise Exception(f'Expected torch.int32 or torch.int64 data, found {x.dtype}.')
    magnitude = torch.abs(x) >> bits
    return (torch.sign(x) * magnitude).to(x.dtype)
