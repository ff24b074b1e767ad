"""Shift along the time axis on the GPU.

Interface of lava.lib.dl.slayer.utils.time.shift (utils/time/shift.py:94-143
in the reference); the body is slayer_shift of libslayer_hip.so, one launch
for the whole batch in both the scalar and the per-neuron form.
"""
import numpy as np
import torch

from ... import _native as N


def shift(input, shift_val, sampling_time=1):
    """Move ``input`` by ``int(shift_val / sampling_time)`` steps along its last
    axis (positive = later), filling with zeros.

    ``shift_val`` is a number or one-element tensor (same shift everywhere), or a
    tensor with one entry per neuron of ``input.shape[1:-1]``.
    """
    if input.dim() <= 1:
        raise AssertionError(
            f'Expected input to have at least two dimension. Found {input.shape=}.')
    per_neuron = torch.is_tensor(shift_val) and shift_val.numel() > 1
    if per_neuron and int(np.prod(input.shape[1:-1])) != shift_val.numel():
        raise Exception('Expected spatial dimension of input and shift_val to be same. '
                        f'Found {input.shape=}, {shift_val.shape=}.')
    dev = N.require_gpu(input)
    input = input.contiguous()
    M, T = N.rows_and_steps(input)
    output = torch.empty_like(input)
    if per_neuron:
        lut = shift_val.detach().to(device=dev, dtype=torch.float32).contiguous()
        steps, npb = 0, N.neurons_per_batch(input)
    else:
        if torch.is_tensor(shift_val):
            shift_val = shift_val.item()
        lut, steps, npb = None, int(shift_val / sampling_time), max(M, 1)
    with N.device_guard(dev):
        N.check(N.lib().slayer_shift(
            N.ptr(output), N.ptr(input), N.ptr(lut), steps, float(sampling_time),
            M, npb, T, N.stream_handle()))
    return output
