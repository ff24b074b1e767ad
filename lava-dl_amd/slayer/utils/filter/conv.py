"""Temporal convolution / correlation on the GPU.

Interface of lava.lib.dl.slayer.utils.filter.{conv, corr}
(utils/filter/conv.py:168-223 in the reference); the bodies are slayer_conv /
slayer_corr of libslayer_hip.so.  Each is the other's adjoint, which is how the
autograd link is made.
"""
import torch

from ... import _native as N


def _run(entry, input, filter, sampling_time):
    dev = N.require_gpu(input, filter)
    input, filter = input.contiguous(), filter.contiguous()
    M, T = N.rows_and_steps(input)
    output = torch.empty_like(input)
    with N.device_guard(dev):
        N.check(getattr(N.lib(), entry)(
            N.ptr(output), N.ptr(input), N.ptr(filter), filter.numel(), float(sampling_time),
            M, T, N.stream_handle()))
    return output


def fwd(input, filter, sampling_time=1):
    """Causal: y[t] = Ts * sum_i filter[i] x[t - i]."""
    return _run('slayer_conv', input, filter, sampling_time)


def bwd(input, filter, sampling_time=1):
    """Anti-causal: y[t] = Ts * sum_i filter[i] x[t + i]."""
    return _run('slayer_corr', input, filter, sampling_time)


class _conv(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, filter, sampling_time):
        ctx.save_for_backward(filter)
        ctx.sampling_time = sampling_time
        return fwd(input, filter.detach(), sampling_time)

    @staticmethod
    def backward(ctx, grad_output):
        filter, = ctx.saved_tensors
        if ctx.needs_input_grad[1]:
            print('convolution filter gradient is not implemented.')
        return bwd(grad_output, filter.detach(), ctx.sampling_time), None, None


class _corr(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, filter, sampling_time):
        ctx.save_for_backward(filter)
        ctx.sampling_time = sampling_time
        return bwd(input, filter.detach(), sampling_time)

    @staticmethod
    def backward(ctx, grad_output):
        filter, = ctx.saved_tensors
        if ctx.needs_input_grad[1]:
            print('correlation filter gradient is not implemented.')
        return fwd(grad_output, filter.detach(), ctx.sampling_time), None, None


def conv(input, filter, sampling_time=1):
    """Convolution in time; the last axis of ``input`` is time, ``filter`` is
    flattened to 1-D.  Output has the shape of ``input``.

    Filters of any length are accepted: only the first ``min(K, T)`` taps can meet a sample of a row, and only
    they are read (rows *and* filters longer than 12288 raise).  One deviation from the reference: for filters
    of 9 to 128 taps a non-finite input sample also makes the few neighbouring
    outputs of its row NaN whose window holds it beyond the filter's support (the matrix-core kernel
    multiplies those samples by zero taps instead of skipping them); finite inputs give the same sums."""
    if input.dim() == 1:
        input = input.reshape(1, -1)
    return _conv.apply(input, filter.flatten(), sampling_time)


def corr(input, filter, sampling_time=1):
    """Correlation in time (the adjoint of :func:`conv`)."""
    if input.dim() == 1:
        input = input.reshape(1, -1)
    return _corr.apply(input, filter.flatten(), sampling_time)
