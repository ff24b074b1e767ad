"""Complex (phase-threshold) spike function on the GPU.

Interface of lava.lib.dl.slayer.spike.complex.Spike (spike/complex.py:10-167
in the reference); forward and backward are one fused kernel each
(slayer_cspike_fwd / slayer_cspike_bwd).
"""
import torch

from .. import _native as N
from .spike import _threshold_tensor


def _last_tensor(imag_last, imag):
    M = imag.numel() // imag.shape[-1] if imag.shape[-1] > 0 else 0
    if torch.is_tensor(imag_last):
        last = imag_last.detach().to(device=imag.device, dtype=imag.dtype)
        if last.numel() not in (1, M):
            last = last.expand(imag.shape[:-1])
        return last.contiguous()
    return torch.tensor([imag_last], device=imag.device, dtype=imag.dtype)


def _fwd(real, imag, threshold, imag_last, graded, scale):
    dev = N.require_gpu(real, imag)
    if real.shape != imag.shape:
        raise RuntimeError(f'real/imag shapes differ: {real.shape} vs {imag.shape}')
    real, imag = real.contiguous(), imag.contiguous()
    th = _threshold_tensor(threshold, real)
    last = _last_tensor(imag_last, imag)
    M, T = N.rows_and_steps(real)
    spikes = torch.empty_like(real)
    with torch.cuda.device(dev):
        N.check(N.lib().slayer_cspike_fwd(
            N.ptr(spikes), N.ptr(real), N.ptr(imag), N.ptr(th), th.numel(),
            N.ptr(last), last.numel(), 1 if graded else 0, float(scale), M, T, N.stream_handle()))
    return spikes, real, imag, th


def _bwd(grad_out, real, imag, th, tau_rho, scale_rho, graded):
    dev = N.require_gpu(grad_out, real, imag, th)
    grad_out = grad_out.contiguous()
    g_re = torch.empty_like(real)
    g_im = torch.empty_like(imag)
    with torch.cuda.device(dev):
        N.check(N.lib().slayer_cspike_bwd(
            N.ptr(g_re), N.ptr(g_im), N.ptr(grad_out), N.ptr(real), N.ptr(imag), N.ptr(th), th.numel(),
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
        spikes, real_c, imag_c, th = _fwd(real, imag, threshold, imag_last, graded, scale)
        ctx.save_for_backward(real_c, imag_c, th)
        ctx.tau_rho, ctx.scale_rho, ctx.graded = float(tau_rho), float(scale_rho), graded
        return spikes

    @staticmethod
    def backward(ctx, grad_output):
        real, imag, th = ctx.saved_tensors
        g_re, g_im = _bwd(grad_output, real, imag, th, ctx.tau_rho, ctx.scale_rho, ctx.graded)
        return g_re, g_im, None, None, None, None, None, None
