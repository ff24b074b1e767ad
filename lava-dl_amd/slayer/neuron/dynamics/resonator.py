"""Resonator dynamics on the GPU.

Interface of lava.lib.dl.slayer.neuron.dynamics.resonator
(neuron/dynamics/resonator.py:49-174 in the reference); the body is
slayer_res_fwd / slayer_res_bwd of libslayer_hip.so.
"""
import torch

from ... import _native as N


def dynamics(real_input, imag_input, sin_decay, cos_decay, real_state, imag_state,
             w_scale, threshold=None, debug=False):
    """z[t] = (cos_decay + i sin_decay)/4096 * z[t-1] + x[t] in 12-bit fixed
    point on the (real, imag) pair.  With a threshold, a step whose imaginary
    part reaches it resets real to 0 and imag to just below the threshold
    (Izhikevich-style).

    Returns
    -------
    (real, imag) : tensors shaped like the inputs.
    """
    if threshold is None:
        threshold = -1
    if not debug and not N.wants_grad(real_input, imag_input, sin_decay, cos_decay):
        return _fwd(real_input, imag_input, sin_decay, cos_decay, real_state, imag_state,
                    threshold, w_scale)                                  # skip the autograd node
    _ResDynamics.DEBUG = debug
    return _ResDynamics.apply(real_input, imag_input, sin_decay, cos_decay,
                              real_state, imag_state, threshold, w_scale)


def persistent_real_state(real_state, spike):
    """Real state to carry over when the last step spiked (reset to 0)."""
    spike = (spike > 0).to(real_state.dtype)
    return real_state * (1 - spike)


def persistent_imag_state(imag_state, spike, threshold, scale):
    """Imaginary state to carry over when the last step spiked."""
    spike = (spike > 0).to(imag_state.dtype)
    return spike * (threshold - 1 / scale) + (1 - spike) * imag_state


def _fwd(real_input, imag_input, sin_decay, cos_decay, real_state, imag_state, threshold, w_scale,
         entry='slayer_res_fwd'):
    dev = N.require_gpu(real_input, imag_input, sin_decay, cos_decay, real_state, imag_state)
    if real_input.shape != imag_input.shape:
        raise RuntimeError(f'real/imag input shapes differ: {real_input.shape} vs {imag_input.shape}')
    if sin_decay.numel() != cos_decay.numel():
        raise RuntimeError('sin_decay and cos_decay must have the same number of elements')
    real_input, imag_input = real_input.contiguous(), imag_input.contiguous()
    sin_decay, cos_decay = sin_decay.contiguous(), cos_decay.contiguous()
    real_state, imag_state = real_state.contiguous(), imag_state.contiguous()
    M, T = N.rows_and_steps(real_input)
    for name, s in (('real_state', real_state), ('imag_state', imag_state)):
        if s.numel() not in (1, M):
            raise RuntimeError(f'{name} has {s.numel()} elements, expected 1 or {M}')
    real = torch.empty_like(real_input)
    imag = torch.empty_like(imag_input)
    with N.device_guard(dev):
        N.check(getattr(N.lib(), entry)(
            N.ptr(real), N.ptr(imag), N.ptr(real_input), N.ptr(imag_input),
            N.ptr(sin_decay), N.ptr(cos_decay), N.ptr(real_state), N.ptr(imag_state),
            float(threshold * w_scale), int(w_scale),
            M, N.neurons_per_batch(real_input), sin_decay.numel(),
            real_state.numel(), imag_state.numel(), T, N.stream_handle()))
    return real, imag


def _bwd(grad_real, grad_imag, real, imag, sin_decay, cos_decay, need_decay_grad=True):
    dev = N.require_gpu(grad_real, grad_imag, real, imag, sin_decay, cos_decay)
    grad_real, grad_imag = grad_real.contiguous(), grad_imag.contiguous()
    sin_decay, cos_decay = sin_decay.contiguous(), cos_decay.contiguous()
    M, T = N.rows_and_steps(grad_real)
    g_re_in = torch.empty_like(grad_real)
    g_im_in = torch.empty_like(grad_imag)
    g_sin = g_cos = workspace = None
    if need_decay_grad:
        g_sin = torch.empty(sin_decay.numel(), dtype=torch.float32, device=dev)
        g_cos = torch.empty(cos_decay.numel(), dtype=torch.float32, device=dev)
        workspace = torch.empty(2 * M + 128 * sin_decay.numel(), dtype=torch.float32, device=dev)
    with N.device_guard(dev):
        N.check(N.lib().slayer_res_bwd(
            N.ptr(g_re_in), N.ptr(g_im_in), N.ptr(g_sin), N.ptr(g_cos),
            N.ptr(grad_real), N.ptr(grad_imag), N.ptr(real), N.ptr(imag),
            N.ptr(sin_decay), N.ptr(cos_decay), N.ptr(workspace),
            M, N.neurons_per_batch(grad_real), sin_decay.numel(), T, N.stream_handle()))
    return g_re_in, g_im_in, g_sin, g_cos


def _bwd_naive(grad_real, grad_imag, sin_decay, cos_decay):
    dev = N.require_gpu(grad_real, grad_imag, sin_decay, cos_decay)
    grad_real, grad_imag = grad_real.contiguous(), grad_imag.contiguous()
    M, T = N.rows_and_steps(grad_real)
    g_re_in, g_im_in = torch.empty_like(grad_real), torch.empty_like(grad_imag)
    with N.device_guard(dev):
        N.check(N.lib().slayer_res_bwd_naive(
            N.ptr(g_re_in), N.ptr(g_im_in), N.ptr(grad_real), N.ptr(grad_imag),
            N.ptr(sin_decay.contiguous()), N.ptr(cos_decay.contiguous()),
            M, N.neurons_per_batch(grad_real), sin_decay.numel(), T, N.stream_handle()))
    return g_re_in, g_im_in


def _raise_on_nan(**tensors):
    """The reference aborts the backward pass on NaN (resonator.py:421-439)."""
    for name, t in tensors.items():
        if t is not None and bool(torch.isnan(t).any()):
            raise Exception(f'{name} has NaN.')


class _ResDynamics(torch.autograd.Function):
    DEBUG = False

    @staticmethod
    def forward(ctx, real_input, imag_input, sin_decay, cos_decay, real_state, imag_state,
                threshold, w_scale):
        args = (real_input, imag_input, sin_decay.detach(), cos_decay.detach(),
                real_state.detach(), imag_state.detach(), threshold, w_scale)
        real, imag = _fwd(*args)
        ctx.debug = _ResDynamics.DEBUG
        if ctx.debug:
            re_check, im_check = _fwd(*args, entry='slayer_res_fwd_naive')
            N.raise_on_mismatch('resonator real', real, re_check)
            N.raise_on_mismatch('resonator imag', imag, im_check)
        ctx.save_for_backward(real, imag, sin_decay, cos_decay)
        return real, imag

    @staticmethod
    def backward(ctx, grad_real, grad_imag):
        real, imag, sin_decay, cos_decay = ctx.saved_tensors
        need = ctx.needs_input_grad[2] or ctx.needs_input_grad[3]
        g_re, g_im, g_sin, g_cos = _bwd(grad_real, grad_imag, real, imag,
                                        sin_decay.detach(), cos_decay.detach(), need)
        if ctx.debug:
            c_re, c_im = _bwd_naive(grad_real, grad_imag, sin_decay.detach(), cos_decay.detach())
            N.raise_on_mismatch('resonator grad real', g_re, c_re, rel=N.scan_tolerance(g_re))
            N.raise_on_mismatch('resonator grad imag', g_im, c_im, rel=N.scan_tolerance(g_im))
        _raise_on_nan(grad_real=grad_real, grad_imag=grad_imag, grad_real_input=g_re,
                      grad_imag_input=g_im, grad_sin_decay=g_sin, grad_cos_decay=g_cos)
        if g_sin is not None:
            g_sin = g_sin.reshape(sin_decay.shape)
            g_cos = g_cos.reshape(cos_decay.shape)
        return g_re, g_im, g_sin, g_cos, None, None, None, None
