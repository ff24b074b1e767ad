"""Adaptive resonator dynamics on the GPU.

Interface of lava.lib.dl.slayer.neuron.dynamics.adaptive_resonator
(neuron/dynamics/adaptive_resonator.py:49-200 in the reference); forward is
slayer_adres_fwd, backward is the resonator's slayer_res_bwd.
"""
import torch

from ... import _native as N
from . import resonator as _res
from .adaptive_threshold import persistent_ref_state, persistent_th_state  # noqa: F401  (same helpers)


def dynamics(real_input, imag_input, sin_decay, cos_decay, ref_decay, th_decay,
             real_state, imag_state, ref_state, th_state, th_scale, th0, w_scale, debug=False):
    """Resonator state (no reset) together with an adaptive threshold and a refractory state that
    react to ``imag >= threshold + refractory``.

    Returns
    -------
    (real, imag, threshold, refractory) : tensors shaped like the inputs; only ``real`` and ``imag``
    carry gradients (to the inputs and to sin_decay / cos_decay).
    """
    return _AdResDynamics.apply(real_input, imag_input, sin_decay, cos_decay, ref_decay, th_decay,
                                real_state, imag_state, ref_state, th_state, th_scale, th0, w_scale)


def _fwd(real_input, imag_input, sin_decay, cos_decay, ref_decay, th_decay,
         real_state, imag_state, ref_state, th_state, th_scale, th0, w_scale):
    tensors = [real_input, imag_input, sin_decay, cos_decay, ref_decay, th_decay,
               real_state, imag_state, ref_state, th_state]
    dev = N.require_gpu(*tensors)
    if real_input.shape != imag_input.shape:
        raise RuntimeError(f'real/imag input shapes differ: {real_input.shape} vs {imag_input.shape}')
    if sin_decay.numel() != cos_decay.numel():
        raise RuntimeError('sin_decay and cos_decay must have the same number of elements')
    (real_input, imag_input, sin_decay, cos_decay, ref_decay, th_decay,
     real_state, imag_state, ref_state, th_state) = [t.contiguous() for t in tensors]
    M, T = N.rows_and_steps(real_input)
    for name, s in (('real_state', real_state), ('imag_state', imag_state),
                    ('ref_state', ref_state), ('th_state', th_state)):
        if s.numel() not in (1, M):
            raise RuntimeError(f'{name} has {s.numel()} elements, expected 1 or {M}')
    outs = [torch.empty_like(real_input) for _ in range(4)]
    with N.device_guard(dev):
        N.check(N.lib().slayer_adres_fwd(
            *[N.ptr(o) for o in outs], N.ptr(real_input), N.ptr(imag_input),
            N.ptr(sin_decay), N.ptr(cos_decay), N.ptr(ref_decay), N.ptr(th_decay),
            N.ptr(real_state), N.ptr(imag_state), N.ptr(ref_state), N.ptr(th_state),
            int(th_scale * w_scale), int(th0 * w_scale), int(w_scale),
            M, N.neurons_per_batch(real_input), sin_decay.numel(), ref_decay.numel(), th_decay.numel(),
            real_state.numel(), imag_state.numel(), ref_state.numel(), th_state.numel(),
            T, N.stream_handle()))
    return tuple(outs)


class _AdResDynamics(torch.autograd.Function):
    @staticmethod
    def forward(ctx, real_input, imag_input, sin_decay, cos_decay, ref_decay, th_decay,
                real_state, imag_state, ref_state, th_state, th_scale, th0, w_scale):
        real, imag, threshold, refractory = _fwd(
            real_input, imag_input, sin_decay.detach(), cos_decay.detach(), ref_decay.detach(),
            th_decay.detach(), real_state.detach(), imag_state.detach(), ref_state.detach(),
            th_state.detach(), th_scale, th0, w_scale)
        ctx.save_for_backward(real, imag, sin_decay, cos_decay)
        ctx.mark_non_differentiable(threshold, refractory)
        return real, imag, threshold, refractory

    @staticmethod
    def backward(ctx, grad_real, grad_imag, *_):
        real, imag, sin_decay, cos_decay = ctx.saved_tensors
        need = ctx.needs_input_grad[2] or ctx.needs_input_grad[3]
        g_re, g_im, g_sin, g_cos = _res._bwd(grad_real, grad_imag, real, imag,
                                             sin_decay.detach(), cos_decay.detach(), need)
        _res._raise_on_nan(grad_real=grad_real, grad_imag=grad_imag, grad_real_input=g_re,
                           grad_imag_input=g_im, grad_sin_decay=g_sin, grad_cos_decay=g_cos)
        if g_sin is not None:
            g_sin, g_cos = g_sin.reshape(sin_decay.shape), g_cos.reshape(cos_decay.shape)
        return (g_re, g_im, g_sin, g_cos) + (None,) * 9
