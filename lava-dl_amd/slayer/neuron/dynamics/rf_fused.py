"""Fused resonate-and-fire dynamics + phase-threshold spike on the GPU.

No counterpart module in the reference: one kernel launch per direction for what
``rf.Neuron.forward`` (neuron/rf.py:473-490 in the reference) does with ``resonator.dynamics``
and ``complex.Spike.apply``, with bit-identical results.
"""
import torch

from ... import _native as N
from . import resonator as _res
from . import delays as D


def dynamics(real_input, imag_input, sin_decay, cos_decay, real_state, imag_state, imag_last, w_scale,
             threshold, tau_rho, scale_rho, graded_spike=False, spike_scale=1, delays=None):
    """(real, imag, spike) of an RF neuron (no reset).  ``imag_last`` is the imaginary response before
    the first step (tensor shaped like the states, one element, or a number).  Gradients flow from
    ``spike`` to both inputs and to sin_decay / cos_decay; real and imag are returned detached.
    ``delays`` (a ``delays.Delays``) folds a shift of both inputs and / or a delay of the spikes into the
    kernels; ``spike`` is then the delayed tensor and a fourth result holds the undelayed spike of the last
    step."""
    out_delay = delays.output_delay if delays else None
    res = _RfFused.apply(real_input, imag_input, sin_decay, cos_decay, real_state, imag_state, imag_last,
                         w_scale, threshold, tau_rho, scale_rho, graded_spike, spike_scale, delays, out_delay)
    return res if delays else res[:3]


def spikes(real_input, imag_input, sin_decay, cos_decay, real_state, imag_state, imag_last, w_scale,
           threshold, graded_spike=False, spike_scale=1, delays=None):
    """Inference form: (real_last, imag_last, spike) with only the spikes written per step; no gradient.
    With ``delays`` a fourth result holds the undelayed spike of the last step."""
    with torch.no_grad():
        folded = D.fold(delays, real_input)
        res = _fwd(real_input, imag_input, sin_decay, cos_decay, real_state, imag_state, imag_last, w_scale,
                   threshold, graded_spike is True, spike_scale, spikes_only=True, folded=folded)
        return res + (folded.spike_last,) if folded else res


def _fwd(real_input, imag_input, sin_decay, cos_decay, real_state, imag_state, imag_last, w_scale,
         threshold, graded, spike_scale, spikes_only=False, folded=None):
    """spikes_only: no real / imag traces; the first two results are then real[..., -1], imag[..., -1]."""
    if not torch.is_tensor(imag_last):
        imag_last = torch.tensor([float(imag_last)], dtype=real_input.dtype, device=real_input.device)
    tensors = [real_input, imag_input, sin_decay, cos_decay, real_state, imag_state, imag_last]
    dev = N.require_gpu(*tensors)
    if real_input.shape != imag_input.shape:
        raise RuntimeError(f'real/imag input shapes differ: {real_input.shape} vs {imag_input.shape}')
    real_input, imag_input, sin_decay, cos_decay, real_state, imag_state, imag_last = \
        [t.contiguous() for t in tensors]
    M, T = N.rows_and_steps(real_input)
    for name, s in (('real_state', real_state), ('imag_state', imag_state), ('imag_last', imag_last)):
        if s.numel() not in (1, M):
            raise RuntimeError(f'{name} has {s.numel()} elements, expected 1 or {M}')
    spk = torch.empty_like(real_input)
    real = imag = re_last = im_last = None
    if spikes_only:
        re_last, im_last = (torch.empty(real_input.shape[:-1], dtype=real_input.dtype, device=dev) for _ in range(2))
    else:
        real, imag = torch.empty_like(real_input), torch.empty_like(real_input)
    with N.device_guard(dev):
        N.check(N.lib().slayer_rf_fwd(
            N.ptr(real), N.ptr(imag), N.ptr(spk), N.ptr(re_last), N.ptr(im_last), N.ptr(real_input),
            N.ptr(imag_input),
            N.ptr(sin_decay), N.ptr(cos_decay), N.ptr(real_state), N.ptr(imag_state), N.ptr(imag_last),
            float(threshold), 1 if graded else 0, float(spike_scale), int(w_scale),
            M, N.neurons_per_batch(real_input), sin_decay.numel(),
            real_state.numel(), imag_state.numel(), imag_last.numel(), T, D.ref(folded), N.stream_handle()))
    return (re_last, im_last, spk) if spikes_only else (real, imag, spk)


def _bwd(grad_spikes, real, imag, sin_decay, cos_decay, threshold, tau_rho, scale_rho, graded,
         need_decay_grad=True, folded=None):
    dev = N.require_gpu(grad_spikes, real, imag, sin_decay, cos_decay)
    grad_spikes, sin_decay, cos_decay = grad_spikes.contiguous(), sin_decay.contiguous(), cos_decay.contiguous()
    M, T = N.rows_and_steps(grad_spikes)
    g_re, g_im = torch.empty_like(grad_spikes), torch.empty_like(grad_spikes)
    g_sin = g_cos = workspace = None
    if need_decay_grad:
        g_sin = torch.empty(sin_decay.numel(), dtype=torch.float32, device=dev)
        g_cos = torch.empty(cos_decay.numel(), dtype=torch.float32, device=dev)
        workspace = torch.empty(2 * M + 128 * sin_decay.numel(), dtype=torch.float32, device=dev)
    with N.device_guard(dev):
        N.check(N.lib().slayer_rf_bwd(
            N.ptr(g_re), N.ptr(g_im), N.ptr(g_sin), N.ptr(g_cos), N.ptr(grad_spikes), N.ptr(real), N.ptr(imag),
            N.ptr(sin_decay), N.ptr(cos_decay), float(threshold), float(tau_rho), float(scale_rho),
            1 if graded else 0, N.ptr(workspace),
            M, N.neurons_per_batch(grad_spikes), sin_decay.numel(), T, D.ref(folded), N.stream_handle()))
    return g_re, g_im, g_sin, g_cos


class _RfFused(torch.autograd.Function):
    @staticmethod
    def forward(ctx, real_input, imag_input, sin_decay, cos_decay, real_state, imag_state, imag_last,
                w_scale, threshold, tau_rho, scale_rho, graded, spike_scale, delays, out_delay):
        graded = graded is True
        last = imag_last.detach() if torch.is_tensor(imag_last) else imag_last
        folded = D.fold(delays, real_input)
        real, imag, spk = _fwd(real_input, imag_input, sin_decay.detach(), cos_decay.detach(),
                               real_state.detach(), imag_state.detach(), last, w_scale, threshold, graded,
                               spike_scale, folded=folded)
        want_delay_grad = out_delay is not None and ctx.needs_input_grad[14]
        ctx.save_for_backward(real, imag, sin_decay, cos_decay, spk if want_delay_grad else None)
        ctx.cfg = (float(threshold), float(tau_rho), float(scale_rho), graded)
        ctx.delays = delays if folded else None
        spk_last = folded.spike_last if folded else None
        ctx.mark_non_differentiable(*[t for t in (real, imag, spk_last) if t is not None])
        return real, imag, spk, spk_last

    @staticmethod
    def backward(ctx, _g_re, _g_im, grad_spikes, _g_last):
        real, imag, sin_decay, cos_decay, spk = ctx.saved_tensors
        threshold, tau_rho, scale_rho, graded = ctx.cfg
        need = ctx.needs_input_grad[2] or ctx.needs_input_grad[3]
        grad_spikes = grad_spikes.contiguous()
        folded = D.fold(ctx.delays, grad_spikes, forward=False, delayed_spikes=spk) if ctx.delays else None
        g_re, g_im, g_sin, g_cos = _bwd(grad_spikes, real, imag, sin_decay.detach(), cos_decay.detach(),
                                        threshold, tau_rho, scale_rho, graded, need,
                                        folded)
        _res._raise_on_nan(grad_spikes=grad_spikes, grad_real_input=g_re, grad_imag_input=g_im,
                           grad_sin_decay=g_sin, grad_cos_decay=g_cos)
        if g_sin is not None:
            g_sin, g_cos = g_sin.reshape(sin_decay.shape), g_cos.reshape(cos_decay.shape)
        g_delay = D.delay_gradient(ctx.delays, folded)
        return (g_re, g_im, g_sin, g_cos) + (None,) * 10 + (g_delay,)
