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


# ------------------------------------------------------------------ graded spikes and ALIF neurons
def _alif_setup(seed=11, n=2, c=6, t=60):
    gen = torch.Generator().manual_seed(seed)
    z = torch.randn(n, c, t, generator=gen) * 2
    rec = torch.randint(-40, 41, (c, c), generator=gen).float() / 32
    decays = [torch.tensor([x]) for x in (1024.0, 512.0, 400.0, 800.0)]       # current, voltage, threshold, refractory
    states = [torch.tensor([0.0]), torch.tensor([0.0]), torch.tensor([1.0]), torch.tensor([0.0])]
    return z, rec, decays, states, gen


def test_alif_loop_without_feedback_is_the_plain_alif_chain():
    """One-step calls with the states handed over as float32 = the operators run over the whole sequence
    (whose adaptive threshold is pinned by the reference's own alif vectors)."""
    z, rec, decays, states, _ = _alif_setup()
    spk, vol, theta, last = O.recurrent_alif_fwd(z, torch.zeros_like(rec), decays, states, 0.5, 1.0, 4096)
    cur = O.li_fwd(z, decays[0], states[0], 4096)
    ref_vol = O.li_fwd(cur, decays[1], states[1], 4096)
    th, ref = O.ath_fwd(ref_vol, states[3], decays[3], states[2], decays[2], 0.5, 1.0, 4096)
    ref_spk = O.spike_fwd(ref_vol, th + ref)
    assert 0.02 < float(ref_spk.mean()) < 0.9
    assert torch.equal(vol, ref_vol) and torch.equal(theta, th + ref) and torch.equal(spk, ref_spk)
    assert torch.equal(last[0], cur[..., -1]) and torch.equal(last[1], ref_vol[..., -1])
    assert torch.equal(last[2], O.ath_persistent_th_state(th[..., -1], ref_spk[..., -1], 0.5))
    assert torch.equal(last[3], O.ath_persistent_ref_state(ref[..., -1], ref_spk[..., -1], th[..., -1]))


def test_alif_spike_raises_threshold_and_refractory_of_the_next_step():
    """Hand-computed: no decay at all (decays 0 on threshold and refractory), full decay on current and voltage."""
    z = torch.zeros(1, 1, 4)
    z[0, 0, 0] = 3.0
    z[0, 0, 1] = 3.0
    z[0, 0, 2] = 6.0
    full, none, zero = torch.tensor([4096.0]), torch.tensor([0.0]), torch.tensor([0.0])
    spk, vol, theta, last = O.recurrent_alif_fwd(z, torch.zeros(1, 1), (full, full, none, none),
                                                 (zero, zero, torch.tensor([2.0]), zero), 0.5, 2.0, 4096)
    # step 0: theta = 2 -> spike; threshold 2.5, refractory 4 -> theta 6.5; step 1 and 2 stay below
    assert torch.equal(theta[0, 0], torch.tensor([2.0, 6.5, 6.5, 6.5]))
    assert torch.equal(spk[0, 0], torch.tensor([1.0, 0.0, 0.0, 0.0]))
    assert torch.equal(vol[0, 0], torch.tensor([3.0, 3.0, 6.0, 0.0]))
    assert float(last[2]) == 2.5 and float(last[3]) == 4.0


def test_graded_feedback_carries_the_voltage():
    c, t = 3, 4
    z = torch.zeros(1, c, t)
    z[0, 0, 0] = 5.0                                   # neuron 0 spikes at step 0 with voltage 5
    rec = torch.zeros(c, c)
    rec[1, 0] = 0.25
    full, zero = torch.tensor([4096.0]), torch.tensor([0.0])
    spk, vol, _, _ = O.recurrent_cuba_fwd(z, rec, full, full, zero, zero, 4096, 1.25, graded=True)
    want_vol = torch.zeros(1, c, t)
    want_vol[0, 0, 0] = 5.0
    want_vol[0, 1, 1] = 1.25                           # 0.25 * 5, reaches the threshold itself
    want_vol[0, 1, 2] = 0.0
    assert torch.equal(vol, want_vol)
    want_spk = torch.zeros(1, c, t)
    want_spk[0, 0, 0] = 5.0
    want_spk[0, 1, 1] = 1.25
    assert torch.equal(spk, want_spk)


def test_backward_loop_with_threshold_trace_and_graded_surrogate_is_autograd():
    z, rec, decays, states, gen = _alif_setup(seed=5, c=5, t=14)
    tau, rho = 0.8, 1.3
    for graded in (False, True):
        spk, vol, theta, _ = O.recurrent_alif_fwd(z, rec, decays, states, 0.5, 1.0, 4096, graded=graded)
        assert spk.sum() > 0
        g = torch.rand(z.shape, generator=gen)
        gz, gw = O.recurrent_cuba_bwd(g, spk, vol, rec, theta, tau, rho, graded=graded)
        d = vol.double() - theta.double()
        factor = rho * torch.exp(d.clamp(max=0) / tau) if graded else rho / (2 * tau) * torch.exp(-d.abs() / tau)
        zz = z.double().requires_grad_()
        rr = rec.double().requires_grad_()
        s = torch.zeros(z.shape[0], z.shape[1], dtype=torch.float64)
        outs = []
        for t in range(z.shape[-1]):
            s = _SpikeWithGivenSurrogate.apply(zz[..., t] + s @ rr.t(), spk[..., t].double(), factor[..., t])
            outs.append(s)
        torch.stack(outs, dim=-1).backward(g.double())
        assert torch.allclose(gz.double(), zz.grad, rtol=1e-5, atol=1e-7)
        assert torch.allclose(gw.double(), rr.grad, rtol=1e-5, atol=1e-6)
