"""Spike function with surrogate gradient on the GPU.

Interface of lava.lib.dl.slayer.spike.Spike (spike/spike.py:26-126 in the
reference); forward and backward are one fused kernel each
(slayer_spike_fwd / slayer_spike_bwd).
"""
import torch

from .. import _native as N


def split_threshold(threshold, like):
    """(device tensor or None, scalar value): a python number travels by value, a tensor
    stays on the device (one element, or expanded to the shape of ``like``)."""
    if torch.is_tensor(threshold):
        th = threshold.detach().to(device=like.device, dtype=like.dtype)
        if th.numel() != 1 and th.shape != like.shape:
            th = th.expand(like.shape)
        return th.contiguous(), 0.0
    return None, float(threshold)


def _fwd(voltage, th, th_value, graded, scale):
    dev = N.require_gpu(voltage)
    spikes = torch.empty_like(voltage)
    with N.device_guard(dev):
        N.check(N.lib().slayer_spike_fwd(
            N.ptr(spikes), N.ptr(voltage), N.ptr(th), 0 if th is None else th.numel(), th_value,
            1 if graded else 0, float(scale), voltage.numel(), N.stream_handle()))
    return spikes


def _bwd(grad_spikes, voltage, th, th_value, tau_rho, scale_rho, graded):
    dev = N.require_gpu(grad_spikes, voltage)
    grad_spikes = grad_spikes.contiguous()
    grad_voltage = torch.empty_like(voltage)
    with N.device_guard(dev):
        N.check(N.lib().slayer_spike_bwd(
            N.ptr(grad_voltage), N.ptr(grad_spikes), N.ptr(voltage), N.ptr(th),
            0 if th is None else th.numel(), th_value,
            float(tau_rho), float(scale_rho), 1 if graded else 0, voltage.numel(), N.stream_handle()))
    return grad_voltage


class Spike(torch.autograd.Function):
    """``Spike.apply(voltage, threshold, tau_rho, scale_rho, graded_spike, voltage_last, scale)``

    forward: ``voltage >= threshold`` (times ``voltage / scale`` for graded spikes);
    backward: ``scale_rho / (2 tau_rho) * exp(-|v - th| / tau_rho)`` (binary) or
    ``scale_rho * exp(min(v - th, 0) / tau_rho)`` (graded) times the incoming gradient.
    ``threshold`` is a float or a tensor shaped like ``voltage``.
    """

    @staticmethod
    def forward(ctx, voltage, threshold, tau_rho, scale_rho, graded_spike, voltage_last, scale):
        graded = graded_spike is True
        voltage = voltage.contiguous()
        th, th_value = split_threshold(threshold, voltage)
        spikes = _fwd(voltage, th, th_value, graded, scale)
        ctx.save_for_backward(voltage, th)
        ctx.th_value, ctx.tau_rho, ctx.scale_rho, ctx.graded = th_value, float(tau_rho), float(scale_rho), graded
        return spikes

    @staticmethod
    def backward(ctx, grad_spikes):
        voltage, th = ctx.saved_tensors
        grad = _bwd(grad_spikes, voltage, th, ctx.th_value, ctx.tau_rho, ctx.scale_rho, ctx.graded)
        return grad, None, None, None, None, None, None
