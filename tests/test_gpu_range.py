"""The 32-bit range of the fixed-point states is watched, not assumed: the reference's CPU branch evaluates in int64
(neuron/dynamics/leaky_integrator.py:213, resonator.py:340, adaptive_threshold.py:237-274), the kernels in int32, and
every forward kernel raises a flag before a sum or product can have left 32 bits.  While the flag is clear the
results equal the 64-bit kernels bit for bit; a state driven past the bound raises it in every operator family."""
import pytest
import torch

from tests.util import dev, sparse_input, seed_of

pytestmark = pytest.mark.gpu


@pytest.fixture()
def slayer():
    import lava_dl_amd.slayer as s
    torch.cuda.synchronize()
    s.clear_range_flag()
    yield s
    torch.cuda.synchronize()
    s.clear_range_flag()
    s.range_policy('raise')


def _raised(slayer):
    torch.cuda.synchronize()
    return slayer.clear_range_flag()


def _trips(slayer, call):
    """True when ``call`` raises the flag: either the call itself reports it (the word was already up when the
    wrapper looked, e.g. raised by the entry point on the host) or it is up once the device has finished."""
    try:
        call()
    except OverflowError:
        _raised(slayer)             # workgroups of the call that are still running raise the flag again: wait, then lower it
        return True
    return _raised(slayer)


W = 64


def test_flag_stays_down_just_below_the_bound_and_results_equal_the_64_bit_kernels(slayer):
    """An integrator driven to 0.9 * 2^30: in range, flag down, every bit equal to the 64-bit kernel."""
    L = slayer.neuron.dynamics.leaky_integrator
    T = 256
    x = torch.full((2, 70, T), 0.9 * 2 ** 30 / W / T, device=dev())
    zero = torch.zeros(1, device=dev())
    y = L.dynamics(x, zero, zero, W)
    assert float(y.abs().max()) * W > 0.85 * 2 ** 30
    assert torch.equal(y, L._fwd(x, zero, zero, -1, W, entry='slayer_li_fwd_naive'))
    assert not _raised(slayer)


@pytest.mark.parametrize('shape', [(2, 70, 256), (3, 5, 131), (1, 3, 40), (2, 1100, 320)])
def test_leaky_integrator_raises_the_flag_before_it_overflows(slayer, shape):
    """Whole-quad rows, rows of any length and short rows (three kernels): the state passes 2^30 but not 2^31 --
    nothing has overflowed yet, the results are still exact, and the flag is up."""
    L = slayer.neuron.dynamics.leaky_integrator
    T = shape[-1]
    x = torch.zeros(shape)
    x[-1, -1, :] = 1.5 * 2 ** 30 / W / T                    # one neuron only
    x = x.to(dev())
    zero = torch.zeros(1, device=dev())
    slayer.range_policy('ignore')                            # look at the flag by hand
    y = L.dynamics(x, zero, zero, W)
    assert _raised(slayer)
    assert torch.equal(y, L._fwd(x, zero, zero, -1, W, entry='slayer_li_fwd_naive'))
    assert not _raised(slayer)                               # the 64-bit kernels report nothing
    # the next operator call finds the word raised and reports it
    L.dynamics(x, zero, zero, W)
    torch.cuda.synchronize()
    slayer.range_policy('raise')
    with pytest.raises(OverflowError, match='32-bit range'):
        L.dynamics(x[:1, :1, :8].contiguous(), zero, zero, W)
    assert not slayer.range_flag()                           # reporting it lowers it


def test_range_check_and_policies(slayer):
    L = slayer.neuron.dynamics.leaky_integrator
    zero = torch.zeros(1, device=dev())
    big = torch.full((1, 1, 64), 3.0e7, device=dev())       # decay 0, driven beyond 2^31: sums saturate
    slayer.range_policy('ignore')
    y = L.dynamics(big, zero, zero, W)
    slayer.range_check()                                     # ignored: nothing happens, the flag stays up
    assert slayer.range_flag()
    assert slayer.range_policy('raise') == 'ignore'
    with pytest.raises(OverflowError):
        slayer.range_check()
    assert not slayer.range_flag()
    assert float(y.max()) * W <= 2.0 ** 31                   # saturated at the limit, not wrapped to a negative value
    assert float(y.min()) >= 0
    slayer.range_policy('ignore')
    L.dynamics(big, zero, zero, W)
    torch.cuda.synchronize()
    slayer.range_policy('warn')
    with pytest.warns(RuntimeWarning, match='32-bit range'):
        slayer.range_check()
    slayer.range_policy('raise')
    # an initial state beyond the bound, a decay multiplier beyond +-8191
    assert _trips(slayer, lambda: L.dynamics(big[..., :8] * 0, zero, torch.full((1,), 1.2 * 2 ** 30 / W, device=dev()), W))
    assert _trips(slayer, lambda: L.dynamics(big[..., :8] * 0, torch.full((1,), -5000.0, device=dev()), zero, W))
    assert not _trips(slayer, lambda: L.dynamics(big[..., :8] * 0, torch.full((1,), -4000.0, device=dev()), zero, W))


def test_every_forward_family_reports(slayer):
    D = slayer.neuron.dynamics
    zero, one = torch.zeros(1, device=dev()), torch.ones(1, device=dev())
    T = 128
    ramp = torch.full((2, 6, T), 1.3 * 2 ** 30 / W / T, device=dev())       # integrates to 1.3 * 2^30
    small = torch.full((2, 6, T), 0.01, device=dev())
    d0 = torch.zeros(6, device=dev())

    # adaptive threshold: a threshold state beyond 2^28 / a step that is; a healthy call stays silent
    assert _trips(slayer, lambda: D.adaptive_threshold.dynamics(small, zero, d0, one * (1.5 * 2 ** 28 / W), d0, 0.5, 1.0, W))
    assert _trips(slayer, lambda: D.adaptive_threshold.dynamics(small, zero, d0, one, d0, 1.1 * 2 ** 28 / W, 1.0, W))
    assert not _trips(slayer, lambda: D.adaptive_threshold.dynamics(small, zero, d0, one, d0, 0.5, 1.0, W))
    # resonator: no rotation, no decay (cos = 4096): the real part integrates past 2^29
    sin, cos = torch.zeros(6, device=dev()), torch.full((6,), 4096.0, device=dev())
    assert _trips(slayer, lambda: D.resonator.dynamics(ramp * 0.5, small, sin, cos, zero, zero, W))
    assert not _trips(slayer, lambda: D.resonator.dynamics(ramp * 0.3, small, sin, cos, zero, zero, W))
    # adaptive resonator and phase threshold (float tiles: checked inside the loop)
    assert _trips(slayer, lambda: D.adaptive_resonator.dynamics(ramp * 0.5, small, sin, cos, d0, d0, zero, zero, zero, one, 0.5, 1.0, W))
    assert _trips(slayer, lambda: D.adaptive_phase_th.dynamics(small, small, zero, zero, d0, one * (1.5 * 2 ** 28 / W), d0, 0.5, 1.0, W))
    # fused blocks: current of the CUBA / ALIF block, real part of the RF block
    assert _trips(slayer, lambda: D.cuba_fused.dynamics(ramp, d0, d0 + 4096, zero, zero, W, 1.0e9, 1.0, 1.0, False, 1))
    assert _trips(slayer, lambda: D.cuba_fused.spikes(ramp, d0, d0 + 4096, zero, zero, W, 1.0e9, False, 1))
    assert _trips(slayer, lambda: D.alif_fused.dynamics(ramp, d0, d0 + 4096, d0, d0, zero, zero, one, zero, 0.5, 1.0, W, 1.0, 1.0, False, 1))
    assert _trips(slayer, lambda: D.rf_fused.dynamics(ramp * 0.5, small, sin, cos, zero, zero, zero, W, 1.0, 0.5, 10.0, False, 1))
    # ... and stay silent on the same tensors at a tenth of the drive
    D.cuba_fused.dynamics(ramp * 0.1, d0, d0 + 4096, zero, zero, W, 1.0e9, 1.0, 1.0, False, 1)
    D.alif_fused.dynamics(ramp * 0.1, d0, d0 + 4096, d0, d0, zero, zero, one, zero, 0.5, 1.0, W, 1.0, 1.0, False, 1)
    assert not _trips(slayer, lambda: D.rf_fused.dynamics(ramp * 0.1, small, sin, cos, zero, zero, zero, W, 1.0, 0.5, 10.0, False, 1))


def test_large_tensor_kernels_report_too(slayer):
    """The multi-wave kernels of large tensors (several rounds of workgroups) and a single offending neuron."""
    L = slayer.neuron.dynamics.leaky_integrator
    shape = (4, 16, 2048, 300)
    gen = torch.Generator().manual_seed(seed_of('range-large'))
    x = sparse_input(gen, shape).to(dev())
    zero = torch.zeros(1, device=dev())
    d = torch.randint(0, 4096, (16,), generator=gen).float().to(dev())
    assert not _trips(slayer, lambda: L.dynamics(x, d, zero, W))
    d[5] = 0.0
    x[3, 5, 1000, :] = 1.2 * 2 ** 30 / W / 300
    assert _trips(slayer, lambda: L.dynamics(x, d, zero, W))
