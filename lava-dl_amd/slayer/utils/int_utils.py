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


class Q2Zero(torch.autograd.Function):
    """Truncation toward zero of a float tensor with an identity gradient (utils/int_utils.py:35-50
    in the reference; a verification aid, not used by the kernels)."""

    @staticmethod
    def forward(ctx, x):
        return torch.trunc(x).to(torch.int32).to(x.dtype)

    @staticmethod
    def backward(ctx, grad_output):
        return grad_output
