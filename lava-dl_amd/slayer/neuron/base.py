"""Shared machinery of the thin CUBA / ALIF / RF neuron modules.

These modules reproduce what the reference's neuron classes do around the
dynamics kernels (neuron/base.py:60-217, neuron/cuba.py:108-440 in the
reference): parameter scaling and quantisation, lazily shaped state buffers,
persistent state across calls, the threshold epsilon and the surrogate-gradient
constants, and the hardware view of the parameters (cx_* integers, device_params).
"""
import numpy as np
import torch

from ..utils.quantize import quantize

P_SCALE = 1 << 12      # decays are stored as 12-bit integers


def hardware_decay(name):
    """Property returning a decay parameter as the integer(s) the hardware is configured with:
    clamped, rounded, a plain int when shared and an int array per channel otherwise
    (neuron/cuba.py:231-251 in the reference)."""
    def get(self):
        self.clamp()
        val = quantize(getattr(self, name)).cpu().data.numpy().astype(int)
        return val[0] if len(val) == 1 else val
    return property(get, doc=f'{name} as configured on the hardware (12-bit integer).')


class Neuron(torch.nn.Module):
    """Scales, gradient constants, parameter and state book-keeping.

    Sub-classes list their learnable decays in ``self._ranges`` (name -> value or
    [min, max] range, as fractions of 1) and their state buffers in
    ``self._state_init`` (name -> initial value).
    """

    def __init__(self, threshold, tau_grad=1, scale_grad=1, scale=1 << 6, norm=None, dropout=None,
                 shared_param=True, persistent_state=False, requires_grad=False, graded_spike=False):
        super().__init__()
        self.p_scale = P_SCALE
        self.w_scale = int(scale)
        self.s_scale = int(scale) * (1 << 6)
        self._threshold = int(threshold * self.w_scale) / self.w_scale
        self.tau_rho = tau_grad * self._threshold
        self.scale_rho = scale_grad
        self.shared_param = shared_param
        self.persistent_state = persistent_state
        self.requires_grad = requires_grad
        self.graded_spike = graded_spike
        self.norm = self._make_norm(norm)
        self.drop = dropout
        self.debug = False
        self.shape = None
        self.num_neurons = None
        self._ranges = {}
        self._state_init = {}

    def _make_norm(self, norm):
        """Instantiate a normalisation; one that quantises what it subtracts (``pre_hook_fx``) uses this
        neuron's weight quantiser for it (neuron/base.py:127-141 in the reference)."""
        if norm is None:
            return None
        instance = norm()
        if hasattr(instance, 'pre_hook_fx'):
            instance.pre_hook_fx = self.quantize_8bit
        return instance

    # ------------------------------------------------------------------ parameters
    @property
    def threshold(self):
        return self._threshold

    def quantize_8bit(self, weight, descale=False):
        """Weight quantiser to link with a synapse (``synapse.pre_hook_fx = neuron.quantize_8bit``):
        steps of 2 / scale, clamped to the 8-bit range; ``descale`` returns integers."""
        q = quantize(weight, step=2 / self.w_scale).clamp(-256 / self.w_scale, 254 / self.w_scale)
        return q * self.w_scale if descale else q

    # --------------------------------------------------------------- hardware view
    @property
    def scale(self):
        """Factor between this representation of the states and the hardware's."""
        return self.w_scale

    @property
    def weight_exponent(self):
        return int(np.log2(self.s_scale // self.w_scale) - 6)

    @property
    def v_th_mant(self):
        """Threshold mantissa."""
        return int(self.threshold * self.w_scale)

    def _register_decays(self, **decays):
        """Shared: one value each.  Per channel: remember [min, max] (a scalar means +-1 %)
        and draw the values when the channel count is known."""
        for name, value in decays.items():
            if self.shared_param:
                if not np.isscalar(value):
                    raise AssertionError(f'Expected {name} to be a scalar when shared_param is True. '
                                         f'Found {value}.')
                start = value
            else:
                if np.isscalar(value):
                    lo, hi = value * 0.99, value * 1.01
                else:
                    if len(value) != 2:
                        raise AssertionError(f'Expected {name} to be of length 2 i.e. [min, max]. Found {value}.')
                    lo, hi = value
                self._ranges[name] = (lo, hi)
                start = lo
            self.register_parameter(name, torch.nn.Parameter(torch.FloatTensor([self.p_scale * start]),
                                                             requires_grad=self.requires_grad))

    def _register_states(self, **states):
        self._state_init = dict(states)
        for name in states:
            self.register_buffer(name, torch.zeros(1, dtype=torch.float), persistent=False)

    def _draw_per_channel(self, channels, device):
        for name, (lo, hi) in self._ranges.items():
            drawn = lo + (hi - lo) * torch.rand(channels, dtype=torch.float).to(device)
            getattr(self, name).data = self.p_scale * drawn
        self._ranges = {}

    def clamp(self):
        with torch.no_grad():
            for name, p in self.named_parameters(recurse=False):
                p.data.clamp_(0, self.p_scale)

    @property
    def device(self):
        return next(self.parameters()).device

    # ---------------------------------------------------------------------- states
    def _prepare(self, input):
        """First call fixes the neuron shape (and draws per-channel parameters); every call
        makes the state buffers match the batch."""
        if self.shape is None:
            if input.dim() < 3:
                raise AssertionError('Expected input to have at least 3 dimensions: '
                                     f'[Batch, Spatial dims ..., Time]. It\'s shape is {input.shape}.')
            self.shape = input.shape[1:-1]
            self.num_neurons = int(np.prod(self.shape))
            if not self.shared_param:
                self._draw_per_channel(self.shape[0], self.device)
        elif input.shape[1:-1] != self.shape:
            raise AssertionError(f'Input tensor shape ({input.shape}) does not match with '
                                 f'Neuron shape ({self.shape}).')
        buffers = self._buffers
        for name, init in self._state_init.items():
            state = buffers[name]
            if state.shape[0] != input.shape[0]:            # new batch size: start from the initial value
                value = float(init() if callable(init) else init)
                buffers[name] = state = torch.full(input.shape[:-1], value, dtype=state.dtype, device=state.device)
            if state.shape[1:] != self.shape:               # still the one-element buffer: broadcast it
                buffers[name] = state * torch.ones(input.shape[:-1], dtype=state.dtype, device=state.device)
        if self.requires_grad:
            self.clamp()

    def _carry(self, **states):
        """Store the states to carry into the next call (registered buffers; written directly, the
        generic attribute path of torch.nn.Module costs several microseconds per state).  A slice of a
        trace is copied so that the trace can be freed; a tensor of its own is kept as it is."""
        for name, value in states.items():
            self._buffers[name] = value.clone() if value._is_view() else value

    def _q(self, name, fused=False):
        """Integer-valued decay with a straight-through gradient.  ``fused``: for a fused neuron kernel, which
        rounds the decays itself (to nearest, ties to even, as ``quantize`` does); the parameter goes in as it is
        unless a gradient has to reach it, which saves the rounding launch."""
        param = getattr(self, name)
        if fused and not (torch.is_grad_enabled() and param.requires_grad):
            return param
        return quantize(param)
