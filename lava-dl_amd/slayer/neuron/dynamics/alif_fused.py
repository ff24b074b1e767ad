"""Fused adaptive-threshold LIF dynamics + spike on the GPU.

No counterpart module in the reference: one kernel launch per direction for what
``alif.Neuron.forward`` (neuron/alif.py:499-525 and :557-591 in the reference) does with
``leaky_integrator.dynamics`` twice, ``adaptive_threshold.dynamics``, a tensor add and
``Spike.apply``, with bit-identical results.
"""
import torch

from ... import _native as N
from . import delays as D


def dynamics(input, current_decay, voltage_decay, threshold_decay, refractory_decay,
             current_state, voltage_state, threshold_state, refractory_state,
             threshold_step, threshold_base, w_scale, tau_rho, scale_rho, graded_spike=False, spike_scale=1,
             keep_current=True, delays=None):
    """(current, voltage, theta, spike, threshold_last, refractory_last) of an ALIF neuron, where
    ``theta = threshold + refractory`` is what the spike compares the voltage against and the two
    ``*_last`` tensors (shaped like the states) are the threshold and refractory values of the last
    step.  Gradients flow from ``spike`` to ``input`` and to the current / voltage decays (the
    threshold dynamics has none, as in the separate operator); the other outputs are detached.
    With ``keep_current=False`` and decays that do not require a gradient the current trace is neither
    written nor read back and ``current`` holds only the last step, shaped like the states.
    ``delays`` (a ``delays.Delays``) folds a shift of the input and / or a delay of the spikes into the
    kernels; ``spike`` is then the delayed tensor and a seventh result holds the undelayed spike of the last
    step."""
    lean = not keep_current and not (current_decay.requires_grad or voltage_decay.requires_grad)
    out_delay = delays.output_delay if delays else None
    res = _AlifFused.apply(input, current_decay, voltage_decay, threshold_decay, refractory_decay,
                           current_state, voltage_state, threshold_state, refractory_state,
                           threshold_step, threshold_base, w_scale, tau_rho, scale_rho, graded_spike, spike_scale,
                           lean, delays, out_delay)
    return res if delays else res[:6]


def spikes(input, current_decay, voltage_decay, threshold_decay, refractory_decay,
           current_state, voltage_state, threshold_state, refractory_state,
           threshold_step, threshold_base, w_scale, graded_spike=False, spike_scale=1, delays=None):
    """Inference form: (current_last, voltage_last, None, spike, threshold_last, refractory_last) with only
    the spikes written per step; no gradient.  With ``delays`` a seventh result holds the undelayed spike of
    the last step."""
    with torch.no_grad():
        folded = D.fold(delays, input)
        res = _fwd(input, (current_decay, voltage_decay, threshold_decay, refractory_decay),
                   (current_state, voltage_state, threshold_state, refractory_state),
                   threshold_step, threshold_base, w_scale, graded_spike is True, spike_scale, True, True, True,
                   folded=folded)
        return res + (folded.spike_last,) if folded else res


def _fwd(input, decays, states, threshold_step, threshold_base, w_scale, graded, spike_scale, want_last=True,
         lean=False, spikes_only=False, folded=None):
    """decays = (current, voltage, threshold, refractory), states likewise.  lean: no current trace,
    the first result is then current[..., -1].  spikes_only (with lean): no voltage / theta traces
    either; the second result is then voltage[..., -1] and the third None."""
    dev = N.require_gpu(input, *decays, *states)
    input = input.contiguous()
    decays = [d.contiguous() for d in decays]
    states = [s.contiguous() for s in states]
    M, T = N.rows_and_steps(input)
    for name, s in zip(('current_state', 'voltage_state', 'threshold_state', 'refractory_state'), states):
        if s.numel() not in (1, M):
            raise RuntimeError(f'{name} has {s.numel()} elements, expected 1 or {M}')
    if spikes_only and not lean:
        raise RuntimeError('spikes_only implies lean')
    spk = torch.empty_like(input)
    vol, theta = (None, None) if spikes_only else (torch.empty_like(input), torch.empty_like(input))
    cur = None if lean else torch.empty_like(input)
    cur_last = torch.empty(input.shape[:-1], dtype=input.dtype, device=dev) if lean else None
    vol_last = torch.empty(input.shape[:-1], dtype=input.dtype, device=dev) if spikes_only else None
    th_last = ref_last = None
    if want_last:
        th_last = torch.empty(input.shape[:-1], dtype=input.dtype, device=dev)
        ref_last = torch.empty(input.shape[:-1], dtype=input.dtype, device=dev)
    with N.device_guard(dev):
        N.check(N.lib().slayer_alif_fwd(
            N.ptr(cur), N.ptr(vol), N.ptr(theta), N.ptr(spk), N.ptr(cur_last), N.ptr(vol_last), N.ptr(th_last),
            N.ptr(ref_last),
            N.ptr(input),
            *[N.ptr(d) for d in decays], *[N.ptr(s) for s in states],
            int(threshold_step * w_scale), int(threshold_base * w_scale), 1 if graded else 0, float(spike_scale),
            int(w_scale), M, N.neurons_per_batch(input), *[d.numel() for d in decays],
            *[s.numel() for s in states], T, D.ref(folded), N.stream_handle()))
    return (cur_last if lean else cur), (vol_last if spikes_only else vol), theta, spk, th_last, ref_last


def _bwd(grad_spikes, vol, theta, cur, i_decay, v_decay, tau_rho, scale_rho, graded, need_decay_grad=True,
         folded=None):
    dev = N.require_gpu(grad_spikes, vol, theta, i_decay, v_decay) if cur is None else \
        N.require_gpu(grad_spikes, vol, theta, cur, i_decay, v_decay)
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
        N.check(N.lib().slayer_alif_bwd(
            N.ptr(grad_input), N.ptr(g_i), N.ptr(g_v), N.ptr(grad_spikes), N.ptr(vol), N.ptr(theta), N.ptr(cur),
            N.ptr(i_decay), N.ptr(v_decay), float(tau_rho), float(scale_rho), 1 if graded else 0, N.ptr(workspace),
            M, N.neurons_per_batch(grad_spikes), i_decay.numel(), v_decay.numel(), T, D.ref(folded),
            N.stream_handle()))
    return grad_input, g_i, g_v


class _AlifFused(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, i_decay, v_decay, th_decay, ref_decay, i_state, v_state, th_state, ref_state,
                threshold_step, threshold_base, w_scale, tau_rho, scale_rho, graded, spike_scale, lean,
                delays, out_delay):
        graded = graded is True
        folded = D.fold(delays, input)
        outs = _fwd(input, [d.detach() for d in (i_decay, v_decay, th_decay, ref_decay)],
                    [s.detach() for s in (i_state, v_state, th_state, ref_state)],
                    threshold_step, threshold_base, w_scale, graded, spike_scale, True, lean, folded=folded)
        cur, vol, theta, spk, th_last, ref_last = outs
        want_delay_grad = out_delay is not None and ctx.needs_input_grad[18]
        ctx.save_for_backward(None if lean else cur, vol, theta, i_decay, v_decay, spk if want_delay_grad else None)
        ctx.cfg = (float(tau_rho), float(scale_rho), graded)
        ctx.delays = delays if folded else None
        spk_last = folded.spike_last if folded else None
        ctx.mark_non_differentiable(*[t for t in (cur, vol, theta, th_last, ref_last, spk_last) if t is not None])
        return outs + (spk_last,)

    @staticmethod
    def backward(ctx, _g_cur, _g_vol, _g_theta, grad_spikes, _g_th, _g_ref, _g_last):
        cur, vol, theta, i_decay, v_decay, spk = ctx.saved_tensors
        tau_rho, scale_rho, graded = ctx.cfg
        need = (ctx.needs_input_grad[1] or ctx.needs_input_grad[2]) and cur is not None
        grad_spikes = grad_spikes.contiguous()
        folded = D.fold(ctx.delays, grad_spikes, forward=False, delayed_spikes=spk) if ctx.delays else None
        g_in, g_i, g_v = _bwd(grad_spikes, vol, theta, cur, i_decay.detach(), v_decay.detach(),
                              tau_rho, scale_rho, graded, need,
                              folded)
        if g_i is not None:
            g_i, g_v = g_i.reshape(i_decay.shape), g_v.reshape(v_decay.shape)
        g_delay = D.delay_gradient(ctx.delays, folded)
        return (g_in, g_i, g_v) + (None,) * 15 + (g_delay,)
