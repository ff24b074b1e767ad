"""Recurrent spiking layer: ``s[t] = neuron(z[t] + R s[t-1])``.

Interface of lava.lib.dl.slayer.utils.recurrent (utils/recurrent.py:7-112 in the reference).
For a CUBA neuron with binary spikes on the GPU the whole time loop is one kernel launch per
direction (slayer_cuba_recurrent_fwd / _bwd); any other neuron runs the reference's loop of
one-step neuron calls.
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


def _fusable(z, neuron):
    from ..neuron import cuba
    return (type(neuron) is cuba.Neuron and z.is_cuda and z.dim() == 3 and z.dtype == torch.float32
            and neuron.norm is None and neuron.drop is None and not neuron.graded_spike
            and neuron.persistent_state and z.shape[1] <= 1024)


def custom_recurrent(z, neuron, recurrent_synapse):
    """Spikes of the recurrent layer for the dendrite input ``z`` ([N, C, T]).  The neuron must keep
    its state between calls (``persistent_state=True``); its state after the call is that of the
    last step.  Gradients reach ``z`` and the recurrent weights; as in the reference, the state the
    neuron carries from one step to the next is treated as a constant."""
    recurrent_mat = _recurrent_matrix(recurrent_synapse)
    if _fusable(z, neuron):
        return _FusedCubaRecurrent.apply(z, neuron, recurrent_mat)
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


class _FusedCubaRecurrent(torch.autograd.Function):
    @staticmethod
    def forward(ctx, z, neuron, recurrent_mat):
        from ..neuron import cuba
        from ..neuron.dynamics import leaky_integrator
        dev = N.require_gpu(z)
        z = z.detach().contiguous()
        neuron._prepare(z)
        n, c, t = z.shape
        rec = recurrent_mat.detach().to(dev).float().contiguous()
        rec_t = torch.cat([rec.transpose(0, 1), rec.new_zeros(1, c)], dim=0).contiguous()   # + the zero row
        i_decay = neuron._q('current_decay').detach().contiguous()
        v_decay = neuron._q('voltage_decay').detach().contiguous()
        i_state, v_state = neuron.current_state.contiguous(), neuron.voltage_state.contiguous()
        spk, vol = torch.empty_like(z), torch.empty_like(z)
        cur_last, vol_last = torch.empty_like(i_state), torch.empty_like(v_state)
        threshold = neuron.threshold + neuron.threshold_eps
        with torch.cuda.device(dev):
            N.check(N.lib().slayer_cuba_recurrent_fwd(
                N.ptr(spk), N.ptr(vol), N.ptr(cur_last), N.ptr(vol_last), N.ptr(z), N.ptr(rec_t),
                N.ptr(i_decay), N.ptr(v_decay), N.ptr(i_state), N.ptr(v_state),
                float(threshold), int(neuron.s_scale), n, c, i_decay.numel(), v_decay.numel(),
                i_state.numel(), v_state.numel(), t, N.stream_handle()))
        neuron.current_state = cur_last
        neuron.voltage_state = leaky_integrator.persistent_state(vol_last, spk[..., -1]).detach().clone()
        ctx.save_for_backward(vol, spk, rec)
        ctx.cfg = (float(threshold), float(neuron.tau_rho * cuba.TAU_RHO_MULT),
                   float(neuron.scale_rho * cuba.SCALE_RHO_MULT))
        return spk

    @staticmethod
    def backward(ctx, grad_x):
        vol, spk, rec = ctx.saved_tensors
        threshold, tau_rho, scale_rho = ctx.cfg
        dev = N.require_gpu(grad_x)
        grad_x = grad_x.contiguous()
        n, c, t = grad_x.shape
        grad_z = torch.empty_like(grad_x)
        with torch.cuda.device(dev):
            N.check(N.lib().slayer_cuba_recurrent_bwd(
                N.ptr(grad_z), N.ptr(grad_x), N.ptr(vol), N.ptr(rec), threshold, tau_rho, scale_rho,
                n, c, t, N.stream_handle()))
        return grad_z, None, _weight_gradient(grad_z, spk)
