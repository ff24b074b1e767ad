"""Sigma decoder on the GPU.

Interface of lava.lib.dl.slayer.dendrite.Sigma (dendrite/sigma.py:10-77 in the
reference, which calls torch.cumsum); the running sum is slayer_cumsum of
libslayer_hip.so: sequential float32 adds per neuron, so the result does not
depend on how a library scan happens to group the terms.
"""
import torch

from .. import _native as N


def _cumsum(input, state=None, reverse=False):
    dev = N.require_gpu(input) if state is None else N.require_gpu(input, state)
    input = input.contiguous()
    state = None if state is None else state.contiguous()
    M, T = N.rows_and_steps(input)
    output = torch.empty_like(input)
    with N.device_guard(dev):
        N.check(N.lib().slayer_cumsum(N.ptr(output), N.ptr(input), N.ptr(state),
                                      0 if state is None else state.numel(), 1 if reverse else 0,
                                      M, T, N.stream_handle()))
    return output


class _RunningSum(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, state):
        return _cumsum(input, state)

    @staticmethod
    def backward(ctx, grad_output):
        return _cumsum(grad_output, None, reverse=True), None


class Sigma(torch.nn.Module):
    """Accumulates delta events back into a signal: ``y[t] = y[t-1] + x[t]``; with
    ``persistent_state`` the sum continues from the previous call."""

    def __init__(self, persistent_state=False):
        super().__init__()
        self.persistent_state = persistent_state
        self.shape = None
        self.register_buffer('pre_state', torch.zeros(1, dtype=torch.float), persistent=False)

    def forward(self, input):
        if self.shape is None:
            if input.dim() < 3:
                raise AssertionError('Expected input to have at least 3 dimensions: '
                                     f'[Batch, Spatial dims ..., Time]. It\'s shape is {input.shape}.')
            self.shape = input.shape[1:-1]
        elif input.shape[1:-1] != self.shape:
            raise AssertionError(f'Input tensor shape ({input.shape}) does not match with '
                                 f'Neuron shape ({self.shape}).')
        if self.pre_state.shape[0] != input.shape[0]:
            self.pre_state = torch.zeros(input.shape[:-1], dtype=self.pre_state.dtype, device=self.pre_state.device)
        if not self.persistent_state:
            return _RunningSum.apply(input, None)
        output = _RunningSum.apply(input, self.pre_state)
        self.pre_state = output[..., -1].detach().clone()
        return output

    @property
    def device_params(self):
        return {'type': 'SDNN', 'sigma_output': True}
