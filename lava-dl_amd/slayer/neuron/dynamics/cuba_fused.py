"""Fused CUBA neuron dynamics + spike on the GPU.

No counterpart module in the reference: it does in one kernel launch per direction what
``cuba.Neuron.forward`` (neuron/cuba.py:423-440 in the reference) does with
``leaky_integrator.dynamics`` twice and ``Spike.apply``, with bit-identical results, reading the
input once and never re-reading the intermediate current and voltage traces.
"""
import torch

from ... import _native as N
from . import delays as D


def dynamics(input, current_decay, voltage_decay, current_state, voltage_state, w_scale, threshold,
             tau_rho, scale_rho, graded_spike=False, spike_scale=1, keep_current=True, delays=None):
    """(current, voltage, spike) of a CUBA neuron.

    ``delays`` (a ``delays.Delays``) folds a shift of the input and / or a delay of the spikes into the
    kernels: the neuron sees ``shift(input, input_shift)``, ``spike`` is the delayed spike tensor and a
    fourth result holds the undelayed spike of the last step; current and voltage stay undelayed.

    With ``keep_current=False`` and decays that do not require a gradient the current trace is
    neither written nor read back (24 instead of 32 bytes per neuron-timestep for forward plus
    backward) and ``current`` holds only the last step, shaped like the states.

    ``threshold`` is used both for the voltage reset (compared in integer state units, as
    ``leaky_integrator.dynamics`` does) and for the spike (compared on the float32 voltage, as
    ``Spike`` does).  Gradients flow from ``spike`` to ``input`` and to both decays; the returned
    current and voltage traces are detached.
    """
    lean = not keep_current and not (current_decay.requires_grad or voltage_decay.requires_grad)
    out_delay = delays.output_delay if delays else None
    res = _CubaFused.apply(input, current_decay, voltage_decay, current_state, voltage_state,
                           w_scale, threshold, tau_rho, scale_rho, graded_spike, spike_scale, lean, delays, out_delay)
    return res if delays else res[:3]


def spikes(input, current_decay, voltage_decay, current_state, voltage_state, w_scale, threshold,
           graded_spike=False, spike_scale=1, delays=None):
    """Inference form: (current_last, voltage_last, spike) with only the spikes written per step
    (8 bytes per neuron-timestep); no gradient.  With ``delays`` a fourth result holds the undelayed
    spike of the last step."""
    with torch.no_grad():
        folded = D.fold(delays, input)
        res = _fwd(input, current_decay, voltage_decay, current_state, voltage_state, w_scale, threshold,
                   graded_spike is True, spike_scale, lean=True, spikes_only=True, folded=folded)
        return res + (folded.spike_last,) if folded else res


def _fwd(input, i_decay, v_decay, i_state, v_state, w_scale, threshold, graded, spike_scale, lean=False,
         spikes_only=False, folded=None):
    """lean: no current trace; the first result is then current[..., -1].  spikes_only (with lean):
    no voltage trace either; the second result is then voltage[..., -1]."""
    dev = N.require_gpu(input, i_decay, v_decay, i_state, v_state)
    input, i_decay, v_decay = input.contiguous(), i_decay.contiguous(), v_decay.contiguous()
    i_state, v_state = i_state.contiguous(), v_state.contiguous()
    M, T = N.rows_and_steps(input)
    for name, s in (('current_state', i_state), ('voltage_state', v_state)):
        if s.numel() not in (1, M):
            raise RuntimeError(f'{name} has {s.numel()} elements, expected 1 or {M}')
    if spikes_only and not lean:
        raise RuntimeError('spikes_only implies lean')
    spk = torch.empty_like(input)
    vol = None if spikes_only else torch.empty_like(input)
    cur = None if lean else torch.empty_like(input)
    cur_last = torch.empty(input.shape[:-1], dtype=input.dtype, device=dev) if lean else None
    vol_last = torch.empty(input.shape[:-1], dtype=input.dtype, device=dev) if spikes_only else None
    with N.device_guard(dev):
        N.check(N.lib().slayer_cuba_fwd(
            N.ptr(cur), N.ptr(vol), N.ptr(spk), N.ptr(cur_last), N.ptr(vol_last), N.ptr(input),
            N.ptr(i_decay), N.ptr(v_decay),
            N.ptr(i_state), N.ptr(v_state), float(threshold * w_scale), float(threshold),
            1 if graded else 0, float(spike_scale), int(w_scale),
            M, N.neurons_per_batch(input), i_decay.numel(), v_decay.numel(),
            i_state.numel(), v_state.numel(), T, D.ref(folded), N.stream_handle()))
    return (cur_last if lean else cur), (vol_last if spikes_only else vol), spk


def _bwd(grad_spikes, vol, cur, i_decay, v_decay, threshold, tau_rho, scale_rho, graded, need_decay_grad=True,
         folded=None):
    dev = N.require_gpu(grad_spikes, vol, i_decay, v_decay) if cur is None else \
        N.require_gpu(grad_spikes, vol, cur, i_decay, v_decay)
    if cur is None and need_decay_grad:
        raise RuntimeError('the decay gradients need the current trace')
    grad_spikes, i_decay, v_decay = grad_spikes.contiguous(), i_decay.contiguous(), v_decay.contiguous()
    M, T = N.rows_and_steps(grad_spikes)
    grad_input = torch.empty_like(grad_spikes)
    g_i = g_v = workspace = None
    if need_decay_grad:
        g_i = torch.empty(i_decay.numel(), dtype=torch.float32, device=dev)
        g_v = torch.empty(v_decay.numel(), dtype=torch.float32, device=dev)
        workspace = torch.empty(2 * M + 64 * (i_decay.numel() + v_decay.numel()), dtype=torch.float32, device=dev)
    with N.device_guard(dev):
        N.check(N.lib().slayer_cuba_bwd(
            N.ptr(grad_input), N.ptr(g_i), N.ptr(g_v), N.ptr(grad_spikes), N.ptr(vol), N.ptr(cur),
            N.ptr(i_decay), N.ptr(v_decay), float(threshold), float(tau_rho), float(scale_rho),
            1 if graded else 0, N.ptr(workspace),
            M, N.neurons_per_batch(grad_spikes), i_decay.numel(), v_decay.numel(), T, D.ref(folded),
            N.stream_handle()))
    return grad_input, g_i, g_v


class _CubaFused(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, i_decay, v_decay, i_state, v_state, w_scale, threshold, tau_rho, scale_rho,
                graded, spike_scale, lean, delays, out_delay):
        graded = graded is True
        folded = D.fold(delays, input)
        cur, vol, spk = _fwd(input, i_decay.detach(), v_decay.detach(), i_state.detach(), v_state.detach(),
                             w_scale, threshold, graded, spike_scale, lean, folded=folded)
        want_delay_grad = out_delay is not None and ctx.needs_input_grad[13]
        ctx.save_for_backward(None if lean else cur, vol, i_decay, v_decay, spk if want_delay_grad else None)
        ctx.cfg = (float(threshold), float(tau_rho), float(scale_rho), graded)
        ctx.delays = delays if folded else None
        spk_last = folded.spike_last if folded else None
        ctx.mark_non_differentiable(*[t for t in (cur, vol, spk_last) if t is not None])
        return cur, vol, spk, spk_last

    @staticmethod
    def backward(ctx, _g_cur, _g_vol, grad_spikes, _g_last):
        cur, vol, i_decay, v_decay, spk = ctx.saved_tensors
        threshold, tau_rho, scale_rho, graded = ctx.cfg
        need = (ctx.needs_input_grad[1] or ctx.needs_input_grad[2]) and cur is not None
        grad_spikes = grad_spikes.contiguous()
        folded = D.fold(ctx.delays, grad_spikes, forward=False, delayed_spikes=spk) if ctx.delays else None
        g_in, g_i, g_v = _bwd(grad_spikes, vol, cur, i_decay.detach(), v_decay.detach(),
                              threshold, tau_rho, scale_rho, graded, need,
                              folded)
        if g_i is not None:
            g_i, g_v = g_i.reshape(i_decay.shape), g_v.reshape(v_decay.shape)
        g_delay = D.delay_gradient(ctx.delays, folded)
        return (g_in, g_i, g_v) + (None,) * 10 + (g_delay,)
