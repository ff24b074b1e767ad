"""Pins of the oracle's recurrent-layer restatement (oracle.recurrent_cuba_fwd / _bwd), on the CPU.

The reference holds no fixture for utils/recurrent.py; its own test compares three implementations
with each other (tests/lava/lib/dl/slayer/utils/test_recurrent.py).  Here the forward loop is pinned
by cases whose answer is known without it, and the backward loop by torch autograd through an
independently written graph with the same 'state is a constant' convention."""
import torch

from oracle import slayer_oracle as O


def _setup(n=2, c=6, t=40, seed=0):
    gen = torch.Generator().manual_seed(seed)
    z = torch.randn(n, c, t, generator=gen)
    rec = torch.randint(-40, 41, (c, c), generator=gen).float() / 32
    d_i, d_v = torch.tensor([1024.0]), torch.tensor([512.0])
    return z, rec, d_i, d_v, gen


def test_without_feedback_the_loop_is_the_plain_neuron():
    z, rec, d_i, d_v, _ = _setup()
    zero = torch.tensor([0.0])
    spk, vol, cs, vs = O.recurrent_cuba_fwd(z, torch.zeros_like(rec), d_i, d_v, zero, zero, 4096, 1.25)
    cur = O.li_fwd(z, d_i, zero, 4096)
    ref_vol = O.li_fwd(cur, d_v, zero, 4096, 1.25)
    ref_spk = O.spike_fwd(ref_vol, 1.25)
    assert ref_spk.sum() > 0
    assert torch.equal(vol, ref_vol) and torch.equal(spk, ref_spk)
    assert torch.equal(cs, cur[..., -1])
    assert torch.equal(vs, O.li_persistent_state(ref_vol[..., -1], ref_spk[..., -1]))


def test_feedback_arrives_one_step_later_through_the_right_weight():
    c, t = 3, 5
    z = torch.zeros(1, c, t)
    z[0, 0, 0] = 5.0                                   # neuron 0 spikes at step 0
    rec = torch.zeros(c, c)
    rec[1, 0] = 0.75                                   # R[out=1][in=0]
    rec[0, 2] = 9.0                                    # must not be used: neuron 2 never spikes
    full = torch.tensor([4096.0])                      # full decay: current = input, voltage = current
    zero = torch.tensor([0.0])
    spk, vol, _, _ = O.recurrent_cuba_fwd(z, rec, full, full, zero, zero, 4096, 1.25)
    want_vol = torch.zeros(1, c, t)
    want_vol[0, 0, 0] = 5.0
    want_vol[0, 1, 1] = 0.75
    assert torch.equal(vol, want_vol)
    assert torch.equal(spk, (want_vol >= 1.25).float())


class _SpikeWithGivenSurrogate(torch.autograd.Function):
    """Forward: the recorded spikes; backward: gradient times the recorded surrogate factor."""

    @staticmethod
    def forward(ctx, dend, spikes, factor):
        ctx.save_for_backward(factor)
        return spikes.clone()

    @staticmethod
    def backward(ctx, grad):
        factor, = ctx.saved_tensors
        return grad * factor, None, None


def test_backward_loop_is_autograd_through_the_unrolled_graph():
    z, rec, d_i, d_v, gen = _setup(n=2, c=5, t=12, seed=3)
    zero = torch.tensor([0.0])
    thr, tau, rho = 1.25, 0.8, 1.3
    spk, vol, _, _ = O.recurrent_cuba_fwd(z, rec, d_i, d_v, zero, zero, 4096, thr)
    g = torch.rand(z.shape, generator=gen)
    gz, gw = O.recurrent_cuba_bwd(g, spk, vol, rec, thr, tau, rho)
    # independent graph: s[t] = Spike(z[t] + s[t-1] R^T), d Spike / d dend = rho/(2 tau) exp(-|v - thr| / tau)
    factor = rho / (2 * tau) * torch.exp(-(vol.double() - thr).abs() / tau)
    zz = z.double().requires_grad_()
    rr = rec.double().requires_grad_()
    s = torch.zeros(z.shape[0], z.shape[1], dtype=torch.float64)
    outs = []
    for t in range(z.shape[-1]):
        s = _SpikeWithGivenSurrogate.apply(zz[..., t] + s @ rr.t(), spk[..., t].double(), factor[..., t])
        outs.append(s)
    torch.stack(outs, dim=-1).backward(g.double())
    assert spk.sum() > 0
    assert torch.allclose(gz.double(), zz.grad, rtol=1e-5, atol=1e-7)
    assert torch.allclose(gw.double(), rr.grad, rtol=1e-5, atol=1e-6)
