"""Delta encoder on the GPU.

Interface of lava.lib.dl.slayer.axon.Delta (axon/delta.py:106-318 in the
reference, where the unit is a python loop over time on every device); forward
and backward are slayer_delta_fwd / slayer_delta_bwd of libslayer_hip.so.
"""
import torch

from .. import _native as N


def _fwd(input, threshold, pre_state, residual_state, error_state, cum_error, quant_step=0.0):
    dev = N.require_gpu(input, threshold, pre_state, residual_state, error_state)
    input = input.contiguous()
    threshold = threshold.contiguous()
    pre_state, residual_state, error_state = (s.contiguous() for s in (pre_state, residual_state, error_state))
    M, T = N.rows_and_steps(input)
    output, delta_input = torch.empty_like(input), torch.empty_like(input)
    residual_out = torch.empty(input.shape[:-1], dtype=input.dtype, device=dev)
    error_out = torch.empty(input.shape[:-1], dtype=input.dtype, device=dev)
    with N.device_guard(dev):
        N.check(N.lib().slayer_delta_fwd(
            N.ptr(output), N.ptr(delta_input), N.ptr(residual_out), N.ptr(error_out),
            N.ptr(input), N.ptr(threshold), N.ptr(pre_state), N.ptr(residual_state), N.ptr(error_state),
            1 if cum_error else 0, float(quant_step),
            M, N.neurons_per_batch(input), threshold.numel(),
            pre_state.numel(), residual_state.numel(), error_state.numel(), T, N.stream_handle()))
    return output, delta_input, residual_out, error_out


def _bwd(grad_output, delta_input, threshold, tau_grad, scale_grad, need_threshold_grad=True):
    dev = N.require_gpu(grad_output, delta_input, threshold)
    grad_output, threshold = grad_output.contiguous(), threshold.contiguous()
    M, T = N.rows_and_steps(grad_output)
    grad_input = torch.empty_like(grad_output)
    grad_threshold = workspace = None
    if need_threshold_grad:
        grad_threshold = torch.empty(threshold.numel(), dtype=torch.float32, device=dev)
        workspace = torch.empty(M + 64 * threshold.numel(), dtype=torch.float32, device=dev)
    with N.device_guard(dev):
        N.check(N.lib().slayer_delta_bwd(
            N.ptr(grad_input), N.ptr(grad_threshold), N.ptr(grad_output), N.ptr(delta_input), N.ptr(threshold),
            N.ptr(workspace), float(tau_grad), float(scale_grad),
            M, N.neurons_per_batch(grad_output), threshold.numel(), T, N.stream_handle()))
    return grad_input, grad_threshold


class _DeltaUnit(torch.autograd.Function):
    """(events, final residual, final error) of the delta unit.  ``quant_step`` > 0 floors the
    events to that grid inside the kernel; the gradient treats the quantiser as identity, as the
    reference's straight-through quantiser does."""

    @staticmethod
    def forward(ctx, input, threshold, pre_state, residual_state, error_state, cum_error,
                tau_grad, scale_grad, quant_step=0.0):
        output, delta_input, residual, error = _fwd(input, threshold.detach(), pre_state, residual_state,
                                                    error_state, cum_error, quant_step)
        ctx.save_for_backward(delta_input, threshold)
        ctx.tau_grad, ctx.scale_grad = float(tau_grad), float(scale_grad)
        ctx.mark_non_differentiable(residual, error)
        return output, residual, error

    @staticmethod
    def backward(ctx, grad_output, *_):
        delta_input, threshold = ctx.saved_tensors
        grad_input, grad_threshold = _bwd(grad_output, delta_input, threshold.detach(), ctx.tau_grad,
                                          ctx.scale_grad, ctx.needs_input_grad[1])
        if grad_threshold is not None:
            grad_threshold = grad_threshold.reshape(threshold.shape)
        return grad_input, grad_threshold, None, None, None, None, None, None, None


class Delta(torch.nn.Module):
    """Delta encoding with a (learnable) threshold: an event carries the accumulated change once it
    reaches the threshold, otherwise the change stays in a residual.  With ``cum_error`` the
    decision is made on the accumulated error instead of the single change.  Events are floored
    to multiples of ``1 / scale``.

    Parameters
    ----------
    threshold : float
    scale : int
        quantisation scale of the events (step 1/scale).
    tau_grad, scale_grad : float
        relaxation and scale of the threshold gradient.
    cum_error, shared_param, persistent_state, requires_grad : bool
    """

    def __init__(self, threshold, scale=(1 << 6), tau_grad=1, scale_grad=1, cum_error=False,
                 shared_param=True, persistent_state=False, requires_grad=False):
        super().__init__()
        self.scale, self.tau_grad, self.scale_grad = scale, tau_grad, scale_grad
        self.cum_error, self.shared_param = cum_error, shared_param
        self.persistent_state, self.requires_grad = persistent_state, requires_grad
        self.shape = None
        for name in ('pre_state', 'residual_state', 'error_state'):
            self.register_buffer(name, torch.zeros(1, dtype=torch.float), persistent=False)
        self.register_parameter('threshold', torch.nn.Parameter(torch.FloatTensor([threshold]),
                                                                requires_grad=requires_grad))

    def clamp(self):
        """Keep the threshold at or above one quantisation step."""
        self.threshold.data.clamp_(1 / self.scale)

    @property
    def device(self):
        return self.threshold.device

    def forward(self, input):
        if self.shape is None:
            if input.dim() < 3:
                raise AssertionError('Expected input to have at least 3 dimensions: '
                                     f'[Batch, Spatial dims ..., Time]. It\'s shape is {input.shape}.')
            self.shape = input.shape[1:-1]
            if not self.shared_param:      # one threshold per channel, shaped [C, 1, ...]
                per_channel = self.threshold.data * torch.ones(self.shape[0], device=self.device)
                self.threshold.data = per_channel.reshape([self.shape[0]] + [1] * (len(self.shape) - 1))
        elif input.shape[1:-1] != self.shape:
            raise AssertionError(f'Input tensor shape ({input.shape}) does not match with'
                                 f'Neuron shape ({self.shape}).')
        if self.pre_state.shape[0] != input.shape[0]:
            for name in ('pre_state', 'residual_state', 'error_state'):
                old = getattr(self, name)
                setattr(self, name, torch.zeros(input.shape[:-1], dtype=old.dtype, device=old.device))
        self.clamp()
        zero = torch.zeros(1, dtype=input.dtype, device=input.device)
        pre, residual = (self.pre_state, self.residual_state) if self.persistent_state else (zero, zero)
        error = self.error_state if self.cum_error else zero
        output, residual_state, error_state = _DeltaUnit.apply(
            input, self.threshold, pre, residual, error, self.cum_error, self.tau_grad, self.scale_grad,
            1 / self.scale)
        if self.persistent_state:
            self.pre_state = input[..., -1].clone().detach()
            self.residual_state = residual_state.clone().detach()
            if self.cum_error:
                self.error_state = error_state.clone().detach()
        return output
