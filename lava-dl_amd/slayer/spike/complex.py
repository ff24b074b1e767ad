"""Complex (phase-threshold) spike function on the GPU.

Interface of lava.lib.dl.slayer.spike.complex.Spike (spike/complex.py:10-167
in the reference); forward and backward are one fused kernel each
(slayer_cspike_fwd / slayer_cspike_bwd).
"""
import torch

from .. import _native as N
from .spike import split_threshold


def _split_last(imag_last, imag):
    M = imag.numel() // imag.shape[-1] if imag.shape[-1] > 0 else 0
    if torch.is_tensor(imag_last):
        last = imag_last.detach().to(device=imag.device, dtype=imag.dtype)
        if last.numel() not in (1, M):
            last = last.expand(imag.shape[:-1])
        return last.contiguous(), 0.0
    return None, float(imag_last)


def _fwd(real, imag, th, th_value, last, last_value, graded, scale):
    dev = N.require_gpu(real, imag)
    if real.shape != imag.shape:
        raise RuntimeError(f'real/imag shapes differ: {real.shape} vs {imag.shape}')
    M, T = N.rows_and_steps(real)
    spikes = torch.empty_like(real)
    with N.device_guard(dev):
        N.check(N.lib().slayer_cspike_fwd(
            N.ptr(spikes), N.ptr(real), N.ptr(imag), N.ptr(th), 0 if th is None else th.numel(), th_value,
            N.ptr(last), 0 if last is None else last.numel(), last_value,
            1 if graded else 0, float(scale), M, T, N.stream_handle()))
    return spikes


def _bwd(grad_out, real, imag, th, th_value, tau_rho, scale_rho, graded):
    dev = N.require_gpu(grad_out, real, imag)
    grad_out = grad_out.contiguous()
    g_re = torch.empty_like(real)
    g_im = torch.empty_like(imag)
    with N.device_guard(dev):
        N.check(N.lib().slayer_cspike_bwd(
            N.ptr(g_re), N.ptr(g_im), N.ptr(grad_out), N.ptr(real), N.ptr(imag), N.ptr(th),
            0 if th is None else th.numel(), th_value,
            float(tau_rho), float(scale_rho), 1 if graded else 0, real.numel(), N.stream_handle()))
    return g_re, g_im


class Spike(torch.autograd.Function):
    """``Spike.apply(real, imag, threshold, tau_rho, scale_rho, graded_spike, imag_last, scale)``

    forward: ``(real >= threshold) & (imag[t-1] < 0) & (imag[t] >= 0)`` with
    ``imag[-1] = imag_last`` (times ``real / scale`` for graded spikes);
    backward: relaxed-delta surrogate in both components.
    """

    @staticmethod
    def forward(ctx, real, imag, threshold, tau_rho, scale_rho, graded_spike, imag_last, scale):
        graded = graded_spike is True
        real, imag = real.contiguous(), imag.contiguous()
        th, th_value = split_threshold(threshold, real)
        last, last_value = _split_last(imag_last, imag)
        spikes = _fwd(real, imag, th, th_value, last, last_value, graded, scale)
        ctx.save_for_backward(real, imag, th)
        ctx.th_value, ctx.tau_rho, ctx.scale_rho, ctx.graded = th_value, float(tau_rho), float(scale_rho), graded
        return spikes

    @staticmethod
    def backward(ctx, grad_output):
        real, imag, th = ctx.saved_tensors
        g_re, g_im = _bwd(grad_output, real, imag, th, ctx.th_value, ctx.tau_rho, ctx.scale_rho, ctx.graded)
        return g_re, g_im, None, None, None, None, None, None
