"""Axonal delay built on the GPU shift and filter kernels.

Interface of lava.lib.dl.slayer.axon.{delay, Delay} (axon/delay.py:10-221 in
the reference).
"""
import numpy as np
import torch

from .. import _native as N
from ..utils.time import shift
from ..utils.filter import conv


def delay(input, delay_val=1, sampling_time=1):
    """Delay ``input`` by ``delay_val`` along time; the gradient is shifted back,
    ``delay_val`` itself gets none."""
    return _delayFunctionNoGradient.apply(input, delay_val, sampling_time)


class Delay(torch.nn.Module):
    """Learnable per-channel axonal delay.

    Parameters
    ----------
    sampling_time : int
    max_delay : int or None
        upper clamp of the delay.
    grad_scale : float
        scale of the delay gradient.
    """

    def __init__(self, sampling_time=1, max_delay=None, grad_scale=1):
        super().__init__()
        self.sampling_time = sampling_time
        self.max_delay = max_delay
        self.grad_scale = grad_scale
        self.register_parameter('delay', torch.nn.Parameter(torch.FloatTensor([0]), requires_grad=True))
        self.init = False
        self.clamp()

    def clamp(self):
        """Keep the delay inside [0, max_delay]."""
        if self.init is True:
            if self.max_delay is None:
                self.delay.data.clamp_(0)
            else:
                self.delay.data.clamp_(0, self.max_delay)

    @property
    def shape(self):
        return None if self.init is False else self.delay.shape

    def per_neuron(self, input):
        """The delays as ``forward`` hands them to the shift: one entry per neuron of ``input.shape[1:-1]``
        (the per-channel parameter repeated over the other neuron axes).  Draws the delays on the first
        call, clamps them, checks the channel count (axon/delay.py:132-176 in the reference)."""
        if self.init is False:
            if input.dim() <= 2:
                raise AssertionError(
                    'Expected input to have at least 3 dimensions: [Batch, Spatial dims ..., Time]. '
                    f"It's shape is {input.shape}.")
            self.delay.data = torch.rand(input.shape[1], dtype=torch.float, device=input.device)
            self.init = True
        self.clamp()
        if self.shape[0] != input.shape[1]:
            raise AssertionError(
                'Expected input to have same number of channels as delays. '
                f'Expected {self.shape[0]}, found {input.shape[1]}.')
        if int(np.prod(input.shape[1:-1])) == self.shape[0]:
            return self.delay
        tile = list(input.shape[1:-1])
        tile[0] = 1
        return self.delay.reshape((-1,) + (1,) * (len(tile) - 1)).repeat(tile)

    def forward(self, input):
        return _delayFunction.apply(input, self.per_neuron(input), self.grad_scale, self.sampling_time)


class _delayFunctionNoGradient(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, delay_val, sampling_time):
        ctx.delay_val, ctx.sampling_time = delay_val, sampling_time
        return shift(input, delay_val, sampling_time)

    @staticmethod
    def backward(ctx, grad_output):
        back = -ctx.delay_val
        return shift(grad_output, back, ctx.sampling_time), None, None


class _delayFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, delay_val, grad_scale, sampling_time):
        output = shift(input, delay_val.data, sampling_time)
        ctx.save_for_backward(output, delay_val.data)
        ctx.grad_scale, ctx.sampling_time = grad_scale, sampling_time
        return output

    @staticmethod
    def backward(ctx, grad_output):
        output, delay_val = ctx.saved_tensors
        ts = ctx.sampling_time
        if delay_val.numel() > 1 and grad_output.numel() > 0:
            grad_input, grad_sum = _delay_bwd(grad_output, output, delay_val, ts)
            return grad_input, grad_sum * ts * ctx.grad_scale, None, None
        # one delay for everything (shift() then divides in double precision), or nothing to do
        # d output / d delay is minus the time derivative: conv with [-1, 1] / Ts gives x[t-1] - x[t]
        diff_filter = torch.tensor([-1, 1], dtype=grad_output.dtype, device=grad_output.device) / ts
        output_diff = conv(output, diff_filter, 1)
        grad_delay = torch.sum(grad_output * output_diff, [0, -1], keepdim=True) \
            .reshape(grad_output.shape[1:-1]) * ts
        return shift(grad_output, -delay_val, ts), grad_delay * ctx.grad_scale, None, None


def _delay_bwd(grad_output, output, delay_val, sampling_time):
    """(grad_input, sum over batch and time of grad_output * d output / d delay) in one pass over
    grad_output and output (slayer_delay_bwd) instead of filter, product, sum and shift."""
    dev = N.require_gpu(grad_output, output)
    grad_output, output = grad_output.contiguous(), output.contiguous()
    M, T = N.rows_and_steps(grad_output)
    npb = N.neurons_per_batch(grad_output)
    if delay_val.numel() != npb:
        raise RuntimeError(f'delay has {delay_val.numel()} elements, expected one per neuron ({npb})')
    lut = delay_val.detach().to(device=dev, dtype=torch.float32).contiguous()
    grad_input = torch.empty_like(grad_output)
    grad_sum = torch.empty(npb, dtype=torch.float32, device=dev)
    workspace = torch.empty(M + 64 * npb, dtype=torch.float32, device=dev)
    with N.device_guard(dev):
        N.check(N.lib().slayer_delay_bwd(
            N.ptr(grad_input), N.ptr(grad_sum), N.ptr(grad_output), N.ptr(output), N.ptr(lut), 0,
            float(sampling_time), N.ptr(workspace), M, npb, T, N.stream_handle()))
    return grad_input, grad_sum.reshape(grad_output.shape[1:-1])
