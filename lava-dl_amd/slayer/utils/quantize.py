"""Straight-through parameter quantiser (utils/quantize.py:18-94 in the reference)."""
from enum import IntEnum, unique

import torch


@unique
class MODE(IntEnum):
    ROUND = 0
    FLOOR = 1


class _StraightThrough(torch.autograd.Function):
    """Snap to a grid of ``step`` in the forward pass, identity in the backward pass."""

    @staticmethod
    def forward(ctx, input, step, use_floor):
        scaled = input / step
        return (torch.floor(scaled) if use_floor else torch.round(scaled)) * step

    @staticmethod
    def backward(ctx, grad_output):
        return grad_output, None, None


def quantize(input, step=1, mode=MODE.ROUND):
    """Quantise ``input`` to multiples of ``step`` (round or floor); gradients pass through."""
    if mode not in (MODE.ROUND, MODE.FLOOR):
        raise ValueError(f'{mode=} is not recognized.')
    if not (torch.is_grad_enabled() and input.requires_grad):      # nothing to pass a gradient to
        snap = torch.floor if mode == MODE.FLOOR else torch.round
        return snap(input) if step == 1 else snap(input / step) * step
    return _StraightThrough.apply(input, step, mode == MODE.FLOOR)


def quantize_hook_fx(x, scale=1 << 6, num_bits=8, descale=False):
    """Synapse pre-hook quantiser (utils/quantize.py:84-115 in the reference): even multiples of
    1 / scale, limited to the signed ``num_bits`` weight range; ``descale`` returns integers."""
    lo = -2 * (1 << num_bits) / scale
    hi = 2 * ((1 << num_bits) - 1) / scale
    q = quantize(x, step=2 / scale).clamp(lo, hi)
    return q * scale if descale else q
