"""Axonal delays folded into the fused neuron kernels.

A block of the reference runs ``neuron -> step_delay -> Delay`` (block/base.py:15-39 and :549-553,
axon/delay.py:10-221) and its input may come through a ``shift`` (utils/time/shift.py:94-143); each
of these is a pass over the tensor of its own.  The fused kernels (``cuba_fused``, ``alif_fused``,
``rf_fused``) can read their input through the shift and store their spikes through the delays
instead, with the same bits as the chain of separate operators.
"""
import ctypes

import numpy as np
import torch

from ... import _native as N


class Delays:
    """What to fold into one fused neuron call.

    Parameters
    ----------
    input_shift : number, tensor or None
        shift of the input in time units, as ``utils.time.shift`` takes it: one value, or one entry per
        neuron of ``input.shape[1:-1]``.  No gradient.
    output_delay : tensor or None
        delay of the spikes in time units, one entry per neuron of ``input.shape[1:-1]`` (what
        ``axon.Delay`` hands to its shift).  When it requires a gradient it receives the one
        ``axon.Delay`` computes, scaled by ``grad_scale``.
    output_steps : int
        whole steps added to every neuron's spike delay (``step_delay`` of a block: 1); not negative.  The
        spikes move by the *sum* ``output_steps + trunc(output_delay / sampling_time)`` of each neuron, in the
        fused kernels and in the separate operators alike (a negative ``output_delay`` entry next to a positive
        ``output_steps`` therefore loses no sample in between); an ``output_head`` or a trained
        ``output_delay`` needs entries that are not negative, as ``axon.Delay`` keeps them.
    output_head : tensor or None
        shaped like the states: the spike that precedes the first one (``step_delay``'s buffer when the
        neuron keeps its state between calls); it lands just before the first spike of this call.
    sampling_time, grad_scale : as in ``axon.Delay``.
    """

    def __init__(self, input_shift=None, output_delay=None, output_steps=0, output_head=None, sampling_time=1,
                 grad_scale=1):
        self.input_shift = input_shift
        self.output_delay = output_delay
        self.output_steps = int(output_steps)
        self.output_head = output_head
        self.sampling_time = sampling_time
        self.grad_scale = grad_scale

        if self.output_steps < 0:
            raise RuntimeError(f'output_steps is a delay in whole steps, it cannot be negative ({self.output_steps})')
        if output_head is not None and self.output_steps != 1:
            raise RuntimeError('output_head is the buffer of a one-step delay: it needs output_steps == 1')

    def __bool__(self):
        return (self.input_shift is not None or self.output_delay is not None or self.output_steps != 0
                or self.output_head is not None)


def needs_grad(delays):
    """True when the spike delay of ``delays`` is being trained."""
    return bool(delays) and torch.is_tensor(delays.output_delay) and delays.output_delay.requires_grad


def _table(value, npb, dev, what):
    """(device table or None, whole steps) for a shift given as a number, a one-element tensor or a
    per-neuron tensor; ``ts`` divides the scalar form in double precision, as ``shift`` does."""
    if value is None:
        return None, None
    if torch.is_tensor(value) and value.numel() > 1:
        if value.numel() != npb:
            raise RuntimeError(f'{what} has {value.numel()} elements, expected one per neuron ({npb})')
        return value.detach().to(device=dev, dtype=torch.float32).contiguous().reshape(-1), None
    return None, (value.item() if torch.is_tensor(value) else value)


class Folded:
    """The C structure for one call, the tensors it points into (kept alive with it) and the tensor that
    receives the last undelayed spike.  A backward call given the delayed spikes of the forward pass also
    asks for the gradient of the spike delay (``grad_sum``: one entry per neuron, summed over batch and time)."""

    def __init__(self, delays, like, forward, delayed_spikes=None):
        dev = like.device
        npb = N.neurons_per_batch(like)
        ts = delays.sampling_time
        in_lut, in_scalar = _table(delays.input_shift, npb, dev, 'input_shift')
        out_lut, out_scalar = _table(delays.output_delay, npb, dev, 'output_delay')
        in_steps = 0 if in_scalar is None else int(in_scalar / ts)
        out_steps = delays.output_steps + (0 if out_scalar is None else int(out_scalar / ts))
        self.spike_last = None
        head = None
        if forward:
            self.spike_last = torch.empty(like.shape[:-1], dtype=torch.float32, device=dev)
            if delays.output_head is not None:
                head = delays.output_head.detach().to(device=dev, dtype=torch.float32).expand(like.shape[:-1]) \
                    .contiguous()
        self.grad_sum = workspace = None
        if delayed_spikes is not None and not forward:
            delayed_spikes = delayed_spikes.contiguous()
            M = delayed_spikes.numel() // max(delayed_spikes.shape[-1], 1)
            self.grad_sum = torch.empty(npb, dtype=torch.float32, device=dev)
            workspace = torch.empty(M + 64 * npb, dtype=torch.float32, device=dev)
        else:
            delayed_spikes = None
        self.keep = (in_lut, out_lut, head, delayed_spikes, workspace)
        self.out_lut, self.out_steps = out_lut, out_steps
        self.struct = N.Delays(N.ptr(in_lut), N.ptr(out_lut), N.ptr(head), N.ptr(self.spike_last),
                               in_steps, out_steps, float(ts),
                               N.ptr(delayed_spikes), N.ptr(self.grad_sum), N.ptr(workspace))

    @property
    def ref(self):
        return ctypes.byref(self.struct)


def fold(delays, like, forward=True, delayed_spikes=None):
    """``Folded`` for a ``Delays`` that folds anything, else None (the kernels then take their plain form).
    ``delayed_spikes`` (backward only): the spikes the forward pass stored, when the spike delay is trained."""
    return Folded(delays, like, forward, delayed_spikes) if delays else None


def delay_gradient(delays, folded):
    """Gradient of ``delays.output_delay`` from what a fused backward call left in ``folded.grad_sum``
    (axon/delay.py:201-221 in the reference: the sum times the sampling time times ``grad_scale``)."""
    if folded is None or folded.grad_sum is None:
        return None
    grad = folded.grad_sum * delays.sampling_time * delays.grad_scale
    if delays.output_delay.numel() == 1:
        grad = grad.sum()
    return grad.reshape(delays.output_delay.shape)


def ref(folded):
    return None if folded is None else folded.ref


def chain_input(delays, input):
    """The input as the neuron sees it, by the separate operator (``axon.delay``)."""
    from ...axon.delay import delay
    if not delays or delays.input_shift is None:
        return input
    return delay(input, delays.input_shift, delays.sampling_time)


def chain_output(delays, spike):
    """The spikes as they leave the block, by the separate operators: ``step_delay`` (block/base.py:15-39),
    then the learnable delay (axon/delay.py:178-221)."""
    from ...axon.delay import delay, _delayFunction
    if not delays:
        return spike
    if delays.output_steps != 0 and delays.output_delay is not None:
        od = delays.output_delay if torch.is_tensor(delays.output_delay) else torch.tensor(float(delays.output_delay))
        if delays.output_head is None and not od.requires_grad:
            # one shift by the sum, as the fused kernels do: two shifts in a row would drop the samples that
            # leave the row in between when the two parts have opposite signs
            steps = delays.output_steps + torch.trunc(od.detach().float() / delays.sampling_time)
            return delay(spike, steps.to(spike.device) if steps.numel() > 1 else float(steps), 1)
        if bool((od.detach() < 0).any()):
            raise RuntimeError('a negative output_delay next to output_steps needs the summed shift, which an '
                               'output_head or a trained output_delay does not take')
    if delays.output_steps != 0:
        spike = delay(spike, delays.output_steps)
        if delays.output_head is not None:
            spike[..., 0] = delays.output_head
    if delays.output_delay is not None:
        spike = _delayFunction.apply(spike, delays.output_delay, delays.grad_scale, delays.sampling_time)
    return spike
