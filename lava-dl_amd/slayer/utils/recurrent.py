"""Recurrent spiking layer: ``s[t] = neuron(z[t] + R s[t-1])``.

Interface of lava.lib.dl.slayer.utils.recurrent (utils/recurrent.py:7-112 in the reference).
For a CUBA or an ALIF neuron on the GPU (binary or graded spikes) the time loop runs inside the library: narrow
layers (and widths up to ``ONE_LAUNCH_MAX`` that are not a multiple of 4) as one kernel launch per direction
(slayer_cuba_recurrent_fwd / slayer_alif_recurrent_fwd / slayer_recurrent_bwd), layers from ``STEPS_FROM`` neurons
on (a multiple of 4 up to 16384) as one launch per time step that multiplies the recurrent matrix with the whole
batch (slayer_*_recurrent_steps_*); any other neuron runs the reference's loop of one-step neuron calls.
"""
import torch

from .. import _native as N


def _recurrent_matrix(recurrent_synapse):
    """[C_out, C_in] weight matrix of the recurrent synapse, through its pre-hook."""
    mat = recurrent_synapse.weight.reshape(recurrent_synapse.weight.shape[:2])
    hook = getattr(recurrent_synapse, 'pre_hook_fx', None)
    return hook(mat) if hook is not None else mat


def custom_recurrent_ground_truth_1(z, neuron, recurrent_synapse):
    """The plain loop: the synapse module computes the feedback, autograd does the rest."""
    x = torch.zeros_like(z)
    spike = torch.zeros(z.shape[:-1], device=z.device)
    for time in range(z.shape[-1]):
        dendrite = z[..., time: time + 1]
        feedback = recurrent_synapse(spike.reshape(dendrite.shape))
        spike = neuron(dendrite + feedback)
        x[..., time: time + 1] = spike
    return x


def custom_recurrent_ground_truth_2(z, neuron, recurrent_synapse):
    """The plain loop with the feedback as a matrix product."""
    x = torch.zeros_like(z)
    recurrent_mat_t = _recurrent_matrix(recurrent_synapse).transpose(0, 1)
    spike = torch.zeros(z.shape[:-1] + (1,), device=z.device)
    for time in range(z.shape[-1]):
        feedback = torch.matmul(spike[..., 0], recurrent_mat_t)
        spike = neuron(torch.unsqueeze(z[..., time] + feedback, dim=-1))
        x[..., time: time + 1] = spike
    return x


ONE_LAUNCH_MAX = 1024       # neurons per sample of the one-launch kernels (one thread per neuron)
STEPS_MAX = 16384           # ... of the launch-per-step kernels (whole quads of neurons)
STEPS_FROM = 256            # width from which a launch per step is the faster form (measured at [32, C, 300])


def _by_steps(c):
    """True for the layer widths that take the launch-per-step kernels."""
    return c % 4 == 0 and c <= STEPS_MAX and (c >= STEPS_FROM or c > ONE_LAUNCH_MAX)


def _fusable(z, neuron):
    from ..neuron import alif, cuba
    if not (type(neuron) in (cuba.Neuron, alif.Neuron) and z.is_cuda and z.dim() == 3 and z.dtype == torch.float32
            and neuron.norm is None and neuron.drop is None and neuron.persistent_state):
        return False
    c = z.shape[1]
    return c <= ONE_LAUNCH_MAX or (_by_steps(c) and z.shape[0] * c < 2 ** 29)


def custom_recurrent(z, neuron, recurrent_synapse):
    """Spikes of the recurrent layer for the dendrite input ``z`` ([N, C, T]).  The neuron must keep
    its state between calls (``persistent_state=True``); its state after the call is that of the
    last step.  Gradients reach ``z`` and the recurrent weights; as in the reference, the state the
    neuron carries from one step to the next is treated as a constant.

    The one-launch kernel adds the feedback row by row in the order the neurons fired, 16 at a time, the
    launch-per-step kernels in a fixed order of their own on the matrix cores (float32), where
    the reference's loop calls ``torch.matmul``.  The sums are the same bits whenever every partial sum
    is exactly representable in float32, which holds for quantised recurrent weights (multiples of a power
    of two of moderate size, what the synapse's ``pre_hook_fx`` quantiser produces).  With unquantised
    weights the sums can differ in the last bit and a dendrite value within that distance of the threshold
    may spike in one and not in the other; no fixture of the reference pins that case."""
    recurrent_mat = _recurrent_matrix(recurrent_synapse)
    if _fusable(z, neuron):
        return _FusedRecurrent.apply(z, neuron, recurrent_mat)
    return CustomRecurrent.apply(z, neuron, recurrent_mat)


class CustomRecurrent(torch.autograd.Function):
    """Loop of one-step neuron calls with a hand-written backward pass (any neuron)."""

    @staticmethod
    def forward(ctx, z, neuron, recurrent_mat):
        z = z.detach().requires_grad_()
        x = torch.zeros_like(z)
        recurrent_mat_t = recurrent_mat.transpose(0, 1).clone().detach().to(z.device)
        ctx.dend_sums, ctx.spikes = [], []
        spike = torch.zeros(z.shape[:-1] + (1,), device=z.device)
        for time in range(z.shape[-1]):
            feedback = torch.matmul(spike[..., 0], recurrent_mat_t)
            with torch.enable_grad():
                dend_sum = (z[..., time] + feedback).detach().requires_grad_()
                spike = neuron(torch.unsqueeze(dend_sum, dim=-1))
            ctx.dend_sums.append(dend_sum)
            ctx.spikes.append(spike)
            x[..., time: time + 1] = spike
        ctx.recurrent_mat = recurrent_mat
        ctx.x = x
        return x.detach()

    @staticmethod
    def backward(ctx, grad_x):
        grad_z = torch.zeros_like(grad_x)
        grad_spike = 0
        for time in range(grad_x.shape[-1])[::-1]:
            grad_spike = grad_spike + grad_x[..., time: time + 1]
            torch.autograd.backward(ctx.spikes[time], grad_spike)
            grad_dend_sum = ctx.dend_sums[time].grad
            grad_spike = torch.unsqueeze(torch.matmul(grad_dend_sum, ctx.recurrent_mat), dim=-1)
            grad_z[..., time] = grad_dend_sum
        return grad_z, None, _weight_gradient(grad_z, ctx.x)


def _weight_gradient(grad_z, x):
    """grad R = sum over batch and time of grad_feedback[t] (outer) spike[t-1]."""
    grad_output = grad_z[..., 1:].transpose(0, 1).reshape(grad_z.shape[1], -1)
    spikes_in = x[..., :-1].transpose(1, 2).reshape(-1, x.shape[1])
    return torch.matmul(grad_output, spikes_in)


def _steps_workspace(n, c, t, with_theta, dev):
    """Scratch memory of a launch-per-step entry point.  The caller holds the tensor until the launches are in the
    stream; torch's allocator hands its memory to later work of the same stream only."""
    floats = N.lib().slayer_recurrent_steps_workspace(n, c, t, 1 if with_theta else 0)
    if floats < 0:
        N.check(int(floats))
    return torch.empty(floats, dtype=torch.float32, device=dev)


class _FusedRecurrent(torch.autograd.Function):
    """The whole time loop of a CUBA or an ALIF layer inside the library: one launch per direction, or one per
    time step for wide layers."""

    @staticmethod
    def forward(ctx, z, neuron, recurrent_mat):
        from ..neuron import alif, cuba
        from ..neuron.dynamics import adaptive_threshold, leaky_integrator
        dev = N.require_gpu(z)
        z = z.detach().contiguous()
        neuron._prepare(z)
        n, c, t = z.shape
        rec = recurrent_mat.detach().to(dev).float().contiguous()
        by_steps = _by_steps(c)
        is_alif = type(neuron) is alif.Neuron
        names = ('current', 'voltage') + (('threshold', 'refractory') if is_alif else ())
        decays = [neuron._q(f'{k}_decay', True).detach().contiguous() for k in names]
        states = [getattr(neuron, f'{k}_state').contiguous() for k in names]
        spk, vol = torch.empty_like(z), torch.empty_like(z)
        theta = torch.empty_like(z) if is_alif else None
        last = [torch.empty_like(s) for s in states]
        graded = 1 if neuron.graded_spike else 0
        if by_steps:
            mat, ws = rec, _steps_workspace(n, c, t, is_alif, dev)
            tail = (N.ptr(ws), ws.numel())
            entry = 'slayer_alif_recurrent_steps_fwd' if is_alif else 'slayer_cuba_recurrent_steps_fwd'
        else:
            mat = torch.cat([rec.transpose(0, 1), rec.new_zeros(1, c)], dim=0).contiguous()   # R^T + the zero row
            tail = ()
            entry = 'slayer_alif_recurrent_fwd' if is_alif else 'slayer_cuba_recurrent_fwd'
        with N.device_guard(dev):
            if is_alif:
                threshold = 0.0
                N.check(getattr(N.lib(), entry)(
                    N.ptr(spk), N.ptr(vol), N.ptr(theta), *[N.ptr(x) for x in last], N.ptr(z), N.ptr(mat),
                    *[N.ptr(d) for d in decays], *[N.ptr(s) for s in states],
                    float(neuron.threshold_step), int(neuron.threshold * neuron.s_scale), graded, 1.0,
                    int(neuron.s_scale), n, c, *[d.numel() for d in decays], *[s.numel() for s in states], t,
                    *tail, N.stream_handle()))
            else:
                threshold = neuron.threshold + neuron.threshold_eps
                N.check(getattr(N.lib(), entry)(
                    N.ptr(spk), N.ptr(vol), *[N.ptr(x) for x in last], N.ptr(z), N.ptr(mat),
                    *[N.ptr(d) for d in decays], *[N.ptr(s) for s in states],
                    float(threshold), graded, 1.0, int(neuron.s_scale), n, c,
                    *[d.numel() for d in decays], *[s.numel() for s in states], t, *tail, N.stream_handle()))
        neuron.current_state = last[0]
        if is_alif:
            neuron.voltage_state = last[1]
            neuron.refractory_state = adaptive_threshold.persistent_ref_state(last[3], spk[..., -1], last[2]).detach()
            neuron.threshold_state = adaptive_threshold.persistent_th_state(
                last[2], spk[..., -1], neuron.threshold_step).detach()
        else:
            neuron.voltage_state = leaky_integrator.persistent_state(last[1], spk[..., -1]).detach().clone()
        mult = alif if is_alif else cuba
        ctx.save_for_backward(vol, spk, rec, *([theta] if is_alif else []))
        ctx.cfg = (float(threshold), float(neuron.tau_rho * mult.TAU_RHO_MULT),
                   float(neuron.scale_rho * mult.SCALE_RHO_MULT), graded)
        return spk

    @staticmethod
    def backward(ctx, grad_x):
        vol, spk, rec, *theta = ctx.saved_tensors
        threshold, tau_rho, scale_rho, graded = ctx.cfg
        dev = N.require_gpu(grad_x)
        grad_x = grad_x.contiguous()
        n, c, t = grad_x.shape
        grad_z = torch.empty_like(grad_x)
        th = N.ptr(theta[0]) if theta else None
        with N.device_guard(dev):
            if _by_steps(c):
                ws = _steps_workspace(n, c, t, bool(theta), dev)
                N.check(N.lib().slayer_recurrent_steps_bwd(
                    N.ptr(grad_z), N.ptr(grad_x), N.ptr(vol), th, N.ptr(rec),
                    threshold, tau_rho, scale_rho, graded, n, c, t, N.ptr(ws), ws.numel(), N.stream_handle()))
            else:
                N.check(N.lib().slayer_recurrent_bwd(
                    N.ptr(grad_z), N.ptr(grad_x), N.ptr(vol), th, N.ptr(rec),
                    threshold, tau_rho, scale_rho, graded, n, c, t, N.stream_handle()))
        return grad_z, None, _weight_gradient(grad_z, spk)
