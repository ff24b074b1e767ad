"""Adaptive threshold and refractory dynamics on the GPU.

Interface of lava.lib.dl.slayer.neuron.dynamics.adaptive_threshold
(neuron/dynamics/adaptive_threshold.py:51-172 in the reference); the body is
slayer_ath_fwd of libslayer_hip.so.  The op has no gradient.
"""
import torch

from ... import _native as N


def dynamics(input, ref_state, ref_decay, th_state, th_decay, th_scale, th0, w_scale, debug=False):
    """Threshold and refractory traces driven by a voltage trace.

    th[t] = (1 - th_decay/4096)(th[t-1] - th0) + th0,  r[t] = (1 - ref_decay/4096) r[t-1]
    in 12-bit fixed point; a step with ``input >= th + r`` then adds ``th_scale``
    to the threshold and ``2 th`` to the refractory state.

    Returns
    -------
    (threshold, refractory) : tensors shaped like ``input`` (values before the
    spike update of each step).
    """
    if not debug and not N.wants_grad(input, ref_state, ref_decay, th_state, th_decay):
        return _fwd(input, ref_state, ref_decay, th_state, th_decay, th_scale, th0, w_scale)   # skip the autograd node
    _ATHDynamics.DEBUG = debug
    return _ATHDynamics.apply(input, ref_state, ref_decay, th_state, th_decay, th_scale, th0, w_scale)


def persistent_ref_state(ref_state, spike, th_state):
    """Refractory state to carry over when the last step spiked."""
    spike = (spike > 0).to(ref_state.dtype)
    return ref_state + 2 * spike * th_state


def persistent_th_state(th_state, spike, th_step):
    """Threshold state to carry over when the last step spiked."""
    spike = (spike > 0).to(th_state.dtype)
    return th_state + spike * th_step


def _fwd(input, ref_state, ref_decay, th_state, th_decay, th_scale, th0, w_scale, entry='slayer_ath_fwd'):
    dev = N.require_gpu(input, ref_state, ref_decay, th_state, th_decay)
    input = input.contiguous()
    ref_state, ref_decay = ref_state.contiguous(), ref_decay.contiguous()
    th_state, th_decay = th_state.contiguous(), th_decay.contiguous()
    M, T = N.rows_and_steps(input)
    for name, s in (('ref_state', ref_state), ('th_state', th_state)):
        if s.numel() not in (1, M):
            raise RuntimeError(f'{name} has {s.numel()} elements, expected 1 or {M}')
    threshold = torch.empty_like(input)
    refractory = torch.empty_like(input)
    with N.device_guard(dev):
        N.check(getattr(N.lib(), entry)(
            N.ptr(threshold), N.ptr(refractory), N.ptr(input),
            N.ptr(ref_state), N.ptr(ref_decay), N.ptr(th_state), N.ptr(th_decay),
            int(th_scale * w_scale), int(th0 * w_scale), int(w_scale),
            M, N.neurons_per_batch(input), ref_decay.numel(), th_decay.numel(),
            ref_state.numel(), th_state.numel(), T, N.stream_handle()))
    return threshold, refractory


class _ATHDynamics(torch.autograd.Function):
    DEBUG = False

    @staticmethod
    def forward(ctx, input, ref_state, ref_decay, th_state, th_decay, th_scale, th0, w_scale):
        args = (input.detach(), ref_state.detach(), ref_decay.detach(), th_state.detach(),
                th_decay.detach(), th_scale, th0, w_scale)
        threshold, refractory = _fwd(*args)
        if _ATHDynamics.DEBUG:
            th_check, ref_check = _fwd(*args, entry='slayer_ath_fwd_naive')
            N.raise_on_mismatch('adaptive_threshold threshold', threshold, th_check)
            N.raise_on_mismatch('adaptive_threshold refractory', refractory, ref_check)
        return threshold, refractory

    @staticmethod
    def backward(*_):
        return None, None, None, None, None, None, None, None
