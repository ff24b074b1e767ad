"""Adaptive phase-threshold dynamics on the GPU.

Interface of lava.lib.dl.slayer.neuron.dynamics.adaptive_phase_th
(neuron/dynamics/adaptive_phase_th.py:51-176 in the reference); the body is
slayer_apth_fwd of libslayer_hip.so.  The op has no gradient.
"""
import torch

from ... import _native as N
from .adaptive_threshold import persistent_ref_state, persistent_th_state  # noqa: F401  (same helpers)


def dynamics(re_input, im_input, im_state, ref_state, ref_decay, th_state, th_decay, th_scale, th0,
             w_scale, debug=False):
    """Threshold and refractory traces of a phase-threshold neuron: the recurrences of
    ``adaptive_threshold.dynamics``, where a step spikes when ``re >= th + r`` while the imaginary
    part crosses zero from below (``im_state`` is the imaginary sample before the first step).

    Returns
    -------
    (threshold, refractory) : tensors shaped like ``re_input``.
    """
    return _APTHDynamics.apply(re_input, im_input, im_state, ref_state, ref_decay, th_state, th_decay,
                               th_scale, th0, w_scale)


def _fwd(re_input, im_input, im_state, ref_state, ref_decay, th_state, th_decay, th_scale, th0, w_scale):
    dev = N.require_gpu(re_input, im_input, im_state, ref_state, ref_decay, th_state, th_decay)
    if re_input.shape != im_input.shape:
        raise RuntimeError(f'real/imag input shapes differ: {re_input.shape} vs {im_input.shape}')
    re_input, im_input = re_input.contiguous(), im_input.contiguous()
    im_state, ref_state, th_state = im_state.contiguous(), ref_state.contiguous(), th_state.contiguous()
    ref_decay, th_decay = ref_decay.contiguous(), th_decay.contiguous()
    M, T = N.rows_and_steps(re_input)
    for name, s in (('im_state', im_state), ('ref_state', ref_state), ('th_state', th_state)):
        if s.numel() not in (1, M):
            raise RuntimeError(f'{name} has {s.numel()} elements, expected 1 or {M}')
    threshold, refractory = torch.empty_like(re_input), torch.empty_like(re_input)
    with N.device_guard(dev):
        N.check(N.lib().slayer_apth_fwd(
            N.ptr(threshold), N.ptr(refractory), N.ptr(re_input), N.ptr(im_input),
            N.ptr(im_state), N.ptr(ref_state), N.ptr(ref_decay), N.ptr(th_state), N.ptr(th_decay),
            int(th_scale * w_scale), int(th0 * w_scale), int(w_scale),
            M, N.neurons_per_batch(re_input), ref_decay.numel(), th_decay.numel(),
            im_state.numel(), ref_state.numel(), th_state.numel(), T, N.stream_handle()))
    return threshold, refractory


class _APTHDynamics(torch.autograd.Function):
    @staticmethod
    def forward(ctx, re_input, im_input, im_state, ref_state, ref_decay, th_state, th_decay,
                th_scale, th0, w_scale):
        return _fwd(re_input.detach(), im_input.detach(), im_state.detach(), ref_state.detach(),
                    ref_decay.detach(), th_state.detach(), th_decay.detach(), th_scale, th0, w_scale)

    @staticmethod
    def backward(*_):
        return (None,) * 10
