"""Neuron -> step_delay -> Delay, the tail of ``AbstractBlock.forward`` (block/base.py:549-553 in the
reference), as one fused kernel launch per direction when the neuron offers it.

Only this tail is here: synapses, masks, weight handling and export of the reference's blocks are not
part of this package.
"""
import torch

from ..axon import delay
from ..neuron.dynamics.delays import Delays


def step_delay(module, x):
    """One step of delay, the time a spike takes from one layer to the next (block/base.py:15-39 in the
    reference).  With a neuron that keeps its state between calls the first sample is the last one of
    the previous call, kept in ``module.delay_buffer``."""
    if hasattr(module, 'delay_buffer') is False:
        module.delay_buffer = None
    persistent_state = hasattr(module, 'neuron') and module.neuron.persistent_state is True
    if module.delay_buffer is not None:
        if module.delay_buffer.shape[0] != x.shape[0]:      # batch mismatch
            module.delay_buffer = None
    if persistent_state:
        delay_buffer = 0 if module.delay_buffer is None else module.delay_buffer
        module.delay_buffer = x[..., -1]
    x = delay(x, 1)
    if persistent_state:
        x[..., 0] = delay_buffer
    return x


def neuron_delay(module, z, fused=True):
    """``x = module.neuron(z)``, then ``step_delay`` when ``module.delay_shift`` is true, then
    ``module.delay`` when it is not None -- what a block does with its synapse's output.  With
    ``fused=True`` and a neuron whose ``forward`` takes ``delays`` (cuba, alif, rf) the two delays are
    folded into the neuron's kernels: the same bits, no pass over the spike tensor of their own."""
    delay_shift = getattr(module, 'delay_shift', False) is True
    axon = getattr(module, 'delay', None)
    neuron = module.neuron
    if not fused or not (delay_shift or axon is not None):
        x = neuron(z)
        if delay_shift:
            x = step_delay(module, x)
        if axon is not None:
            x = axon(x)
        return x
    like = z[0] if isinstance(z, (tuple, list)) else z
    head = None
    persistent_state = neuron.persistent_state is True
    if delay_shift:
        if getattr(module, 'delay_buffer', None) is not None and module.delay_buffer.shape[0] != like.shape[0]:
            module.delay_buffer = None
        if persistent_state:
            head = getattr(module, 'delay_buffer', None)
            if head is None:
                head = torch.zeros(like.shape[:-1], dtype=like.dtype, device=like.device)
    folded = Delays(output_delay=None if axon is None else axon.per_neuron(like),
                    output_steps=1 if delay_shift else 0, output_head=head,
                    sampling_time=1 if axon is None else axon.sampling_time,
                    grad_scale=1 if axon is None else axon.grad_scale)
    x = neuron(z, delays=folded)
    if delay_shift and persistent_state:
        module.delay_buffer = neuron.spike_last
    return x
