"""Leaky integrator dynamics on the GPU.

Interface of lava.lib.dl.slayer.neuron.dynamics.leaky_integrator
(neuron/dynamics/leaky_integrator.py:50-119 in the reference); the body is
slayer_li_fwd / slayer_li_bwd of libslayer_hip.so.
"""
import torch

from ... import _native as N


def dynamics(input, decay, state, w_scale, threshold=None, debug=False):
    """y[t] = (1 - decay/4096) y[t-1] + x[t] in 12-bit fixed point, with an
    optional spike-and-reset at ``threshold``.

    Parameters
    ----------
    input : torch.Tensor
        float32 GPU tensor [N, C, ..., T].
    decay : torch.Tensor
        unscaled integer decay(s): one value (shared), C values (per channel)
        or one per neuron of a batch element.
    state : torch.Tensor
        initial state, one element or shaped like ``input.shape[:-1]``.
    w_scale : int
        scale of the integer state.
    threshold : float or None
        ``None`` disables the reset.
    debug : bool
        also run the independent one-thread-per-neuron kernel (64-bit state) in
        forward and backward and raise if the two results differ in any bit.

    Returns
    -------
    torch.Tensor, same shape as ``input``.
    """
    if threshold is None:
        threshold = -1
    if not debug and not N.wants_grad(input, decay):
        return _fwd(input, decay, state, threshold, w_scale)     # skip the autograd node
    _LIDynamics.DEBUG = debug
    return _LIDynamics.apply(input, decay, state, threshold, w_scale)


def persistent_state(state, spike):
    """State to carry to the next call when the last step spiked (reset to 0)."""
    return state * (spike > 0).logical_not()      # = state * (1 - (spike > 0)): a zero with the state's sign where it spiked


def _fwd(input, decay, state, threshold, w_scale, entry='slayer_li_fwd'):
    dev = N.require_gpu(input, decay, state)
    input, decay, state = input.contiguous(), decay.contiguous(), state.contiguous()
    M, T = N.rows_and_steps(input)
    if state.numel() not in (1, M):
        raise RuntimeError(f'state has {state.numel()} elements, expected 1 or {M}')
    output = torch.empty_like(input)
    with N.device_guard(dev):
        N.check(getattr(N.lib(), entry)(
            N.ptr(output), N.ptr(input), N.ptr(decay), N.ptr(state),
            float(threshold * w_scale), int(w_scale),
            M, N.neurons_per_batch(input), decay.numel(), state.numel(), T, N.stream_handle()))
    return output


def _bwd(grad_output, output, decay, need_decay_grad=True, per_neuron_sums=False):
    """(grad_input, grad_decay).  ``per_neuron_sums`` (without ``need_decay_grad``) returns the per-neuron sums
    the decay gradient is reduced from in place of it: the main kernel alone, no reduction launches."""
    dev = N.require_gpu(grad_output, output, decay)
    grad_output, output, decay = grad_output.contiguous(), output.contiguous(), decay.contiguous()
    M, T = N.rows_and_steps(grad_output)
    grad_input = torch.empty_like(grad_output)
    grad_decay = workspace = None
    if need_decay_grad:
        grad_decay = torch.empty(decay.numel(), dtype=torch.float32, device=dev)
    if need_decay_grad or per_neuron_sums:
        workspace = torch.empty(M + 64 * decay.numel(), dtype=torch.float32, device=dev)
    with N.device_guard(dev):
        N.check(N.lib().slayer_li_bwd(
            N.ptr(grad_input), N.ptr(grad_decay), N.ptr(grad_output), N.ptr(output), N.ptr(decay),
            N.ptr(workspace), M, N.neurons_per_batch(grad_output), decay.numel(), T, N.stream_handle()))
    return grad_input, (workspace[:M] if per_neuron_sums and not need_decay_grad else grad_decay)


def _bwd_naive(grad_output, decay):
    dev = N.require_gpu(grad_output, decay)
    grad_output, decay = grad_output.contiguous(), decay.contiguous()
    M, T = N.rows_and_steps(grad_output)
    grad_input = torch.empty_like(grad_output)
    with N.device_guard(dev):
        N.check(N.lib().slayer_li_bwd_naive(
            N.ptr(grad_input), N.ptr(grad_output), N.ptr(decay), M, N.neurons_per_batch(grad_output),
            decay.numel(), T, N.stream_handle()))
    return grad_input


class _LIDynamics(torch.autograd.Function):
    DEBUG = False

    @staticmethod
    def forward(ctx, input, decay, state, threshold, w_scale):
        output = _fwd(input, decay.detach(), state.detach(), threshold, w_scale)
        ctx.debug = _LIDynamics.DEBUG
        if ctx.debug:
            N.raise_on_mismatch('leaky_integrator forward', output,
                                _fwd(input, decay.detach(), state.detach(), threshold, w_scale,
                                     entry='slayer_li_fwd_naive'))
        ctx.save_for_backward(output, decay)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        output, decay = ctx.saved_tensors
        need = ctx.needs_input_grad[1]
        grad_input, grad_decay = _bwd(grad_output, output, decay.detach(), need)
        if ctx.debug:
            N.raise_on_mismatch('leaky_integrator backward', grad_input, _bwd_naive(grad_output, decay.detach()),
                                rel=N.scan_tolerance(grad_output))
        if grad_decay is not None:
            grad_decay = grad_decay.reshape(decay.shape)
        return grad_input, grad_decay, None, None, None
